// k_copy.hip -- strided N-d data movement for gfx950: Permute (tenferro-prims/src/lib.rs:194-202),
// conj (tenferro-tensor/src/lib.rs:622-658), fill (zeros/ones, :336-347) and ElementwiseMul
// (tenferro-prims/src/lib.rs:241-244).
//
// One kernel family.  The host picks a tile: up to four axes with power-of-two tile extents, chosen so
// that the tile holds a >=512-byte contiguous run on the input side AND on the output side.  A block
// reads the tile in input-memory order (coalesced), parks it in LDS, and writes it in output-memory
// order (coalesced); in-tile coordinates are shifts and masks, the per-block origin is decomposed once.
// HBM-bound: algorithmic bytes = 2 * elements * sizeof(T).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <type_traits>
#include <vector>

#include "internal.hpp"
#include "launch.hpp"

namespace tfh {
namespace {

constexpr int MAXT = 4;    // tile axes
constexpr int MAXG = 16;   // grid axes
constexpr int THREADS = 256;
constexpr int MAXU = 16;   // accesses per thread and side in the large-tile variant

struct CopyArgs {
    const void* in;
    const void* in2;       // second input (elementwise mul)
    void* out;
    int32_t nt, ng;
    int32_t tile_elems;    // product of tile extents (power of two)
    int32_t pad_;
    int64_t ntiles;        // tiles in the whole tensor (the copy kernel's blocks loop over them)
    // fast path: every in-tile offset, taken relative to the lowest address of the tile, fits 32-bit bytes
    int32_t fast32, pad2_;
    int64_t in_rebase, out_rebase;   // lowest in-tile element offset on each side (<= 0)
    int32_t t_text[MAXT];            // tile extent per tile-axis id
    // tile axes in read order (ascending input stride) and in write order (ascending output stride)
    int32_t r_shift[MAXT], r_mask[MAXT], r_id[MAXT];
    int64_t r_si[MAXT];
    int32_t w_shift[MAXT], w_mask[MAXT], w_id[MAXT], w_rpos[MAXT];
    int64_t w_so[MAXT], w_si[MAXT], w_si2[MAXT];
    int64_t t_n[MAXT];     // full extent of tile axis id
    // grid axes (every axis with more than one tile)
    int64_t g_count[MAXG], g_si[MAXG], g_si2[MAXG], g_so[MAXG];
    int32_t g_tid[MAXG];   // tile axis id advanced by this grid axis, or -1
    int32_t g_text[MAXG];  // tile extent of that axis (1 if untiled)
    double alpha_re, alpha_im, beta_re, beta_im;
    int32_t conj, use_beta;
    // large-tile variant: access u of a thread is at tile position (u * threads + tid) * vector length; the part of its
    // offsets that depends on u alone (byte offsets on either side, LDS position of the written element) comes from the
    // host, so a thread works out its own part once instead of sixteen times
    uint32_t u_roff[MAXU], u_woff[MAXU];
    int32_t u_wl[MAXU];
    uint32_t walk_inc[4];   // mixed-radix digits of the block count (the distance between a block's successive tiles)
    uint32_t walk_magic[4]; // floor(2^32 / g_count[g]): the first tile's digits by multiply-high instead of division
    // byte strides of the tile axes in read and in write order and the rebase distances, all modulo 2^32 (in-tile
    // offsets span less than 4 GiB, so wrapped 32-bit sums are exact): a thread's own part of its offsets in a dozen
    // 32-bit multiply-adds
    uint32_t r_sb[MAXT], w_sb[MAXT], in_rebase_b, out_rebase_b;
};

__device__ __forceinline__ int swz(int r) { return r + (r >> 5); }

struct BlockOrigin {
    int64_t in, in2, out;
    int64_t lim[MAXT];  // remaining extent of each tile axis at this block
};

__device__ __forceinline__ int64_t uniform64(int64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)v >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}

__device__ __forceinline__ BlockOrigin block_origin(const CopyArgs& a, uint64_t bid) {
    BlockOrigin o;
    o.in = o.in2 = o.out = 0;
#pragma unroll
    for (int t = 0; t < MAXT; ++t) o.lim[t] = t < a.nt ? a.t_n[t] : 1;
    for (int g = 0; g < a.ng; ++g) {
        uint64_t q = bid / (uint64_t)a.g_count[g];
        int64_t c = (int64_t)(bid - q * (uint64_t)a.g_count[g]);
        bid = q;
        o.in += c * a.g_si[g];
        o.in2 += c * a.g_si2[g];
        o.out += c * a.g_so[g];
        int t = a.g_tid[g];
        if (t >= 0) {
#pragma unroll
            for (int k = 0; k < MAXT; ++k)
                if (k == t) o.lim[k] -= c * a.g_text[g];
        }
    }
    // the tile index is uniform, but the division sequences above run on the vector unit: move the results to
    // scalar registers so a tile origin costs no vector registers
    o.in = uniform64(o.in);
    o.in2 = uniform64(o.in2);
    o.out = uniform64(o.out);
#pragma unroll
    for (int t = 0; t < MAXT; ++t) o.lim[t] = uniform64(o.lim[t]);
    return o;
}

// The tiles a persistent block moves are gridDim.x apart.  Instead of decomposing every tile index by division (64-bit
// divisions run on the vector unit, hundreds of cycles per grid axis between a barrier and the next tile's loads), the
// block keeps the mixed-radix digits of its tile index and adds the digits of gridDim.x with carry: scalar adds and
// compares only.  Digits fit 32 bits (the host takes the fast path only then).
constexpr int WALKG = 4;   // grid axes the walk handles (the host checks)
struct TileWalk {   // (grid axes past a.ng have count 1 and stride 0 on the host side: no conditions in here)
    uint32_t c[WALKG], inc[WALKG];
    __device__ __forceinline__ void start(const CopyArgs& a, uint32_t first) {
#pragma unroll
        for (int g = 0; g < WALKG; ++g) {
            // n >= 1: mulhi(first, floor(2^32 / n)) is the quotient or one less
            const uint32_t n = (uint32_t)a.g_count[g];
            uint32_t q = __umulhi(first, a.walk_magic[g]), rem = first - q * n;
            if (rem >= n) {
                ++q;
                rem -= n;
            }
            c[g] = rem;
            first = q;
            inc[g] = a.walk_inc[g];
        }
    }
    __device__ __forceinline__ void advance(const CopyArgs& a) {
        uint32_t carry = 0;
#pragma unroll
        for (int g = 0; g < WALKG; ++g) {
            const uint32_t n = (uint32_t)a.g_count[g];
            const uint32_t v = c[g] + inc[g] + carry;   // < 2 n
            carry = v >= n ? 1u : 0u;
            c[g] = v >= n ? v - n : v;
        }
    }
    __device__ __forceinline__ void offsets(const CopyArgs& a, int64_t& in, int64_t& out) const {
        in = out = 0;
#pragma unroll
        for (int g = 0; g < WALKG; ++g) {
            in += (int64_t)c[g] * a.g_si[g];
            out += (int64_t)c[g] * a.g_so[g];
        }
    }
};

// ---- element operations -----------------------------------------------------------------------------
template <class V>
struct RawOp {  // bit-exact move
    static constexpr bool kNeedsOld = false;
    __device__ V operator()(V x, V, const CopyArgs&) const { return x; }
};
template <class R>
struct RealOp {  // out = alpha*x + beta*old
    __device__ R operator()(R x, R old, const CopyArgs& a) const {
        R r = (R)a.alpha_re * x;
        if (a.use_beta) r += (R)a.beta_re * old;
        return r;
    }
};
template <class V, class R>
struct CplxOp {  // V = float2/double2
    __device__ V operator()(V x, V old, const CopyArgs& a) const {
        R xr = x.x, xi = a.conj ? -x.y : x.y;
        R ar = (R)a.alpha_re, ai = (R)a.alpha_im;
        V r;
        r.x = ar * xr - ai * xi;
        r.y = ar * xi + ai * xr;
        if (a.use_beta) {
            R br = (R)a.beta_re, bi = (R)a.beta_im;
            r.x += br * old.x - bi * old.y;
            r.y += br * old.y + bi * old.x;
        }
        return r;
    }
};
template <class V>
struct ConjOp {  // bit-exact conj: flip the sign of the imaginary part
    __device__ V operator()(V x, V, const CopyArgs&) const {
        x.y = -x.y;
        return x;
    }
};

template <class V, int N>
struct alignas(sizeof(V) * N) Pack {
    V v[N];
};

__device__ __forceinline__ int64_t pick_lim(const BlockOrigin& o, int id) {
    return id == 0 ? o.lim[0] : id == 1 ? o.lim[1] : id == 2 ? o.lim[2] : o.lim[3];
}

typedef const __attribute__((address_space(1))) char* gcptr;
typedef __attribute__((address_space(1))) char* gmptr;
template <int BYTES> struct RawBits;
template <> struct RawBits<4> { typedef uint32_t type; };
template <> struct RawBits<8> { typedef uint32_t type __attribute__((ext_vector_type(2))); };
template <> struct RawBits<16> { typedef uint32_t type __attribute__((ext_vector_type(4))); };
// Global load/store of a Pack through a uniform base and a 32-bit byte offset (scalar-base addressing).  Every
// byte is touched once, so the accesses carry the non-temporal hint: a plain 16-byte copy of 134 MB measures 6.4 TB/s
// with it against 5.9 TB/s without on this device.
template <class P>
__device__ __forceinline__ P gload_pack(gcptr base, uint32_t off) {
    typedef typename RawBits<sizeof(P)>::type Raw;
    const Raw r = __builtin_nontemporal_load(reinterpret_cast<const __attribute__((address_space(1))) Raw*>(base + off));
    return __builtin_bit_cast(P, r);
}
template <class P>
__device__ __forceinline__ void gstore_pack(gmptr base, uint32_t off, const P& p) {
    typedef typename RawBits<sizeof(P)>::type Raw;
    __builtin_nontemporal_store(__builtin_bit_cast(Raw, p), reinterpret_cast<__attribute__((address_space(1))) Raw*>(base + off));
}

// The same through ordinary pointers (general path).
template <class P>
__device__ __forceinline__ P load_stream(const void* p) {
    typedef typename RawBits<sizeof(P)>::type Raw;
    return __builtin_bit_cast(P, __builtin_nontemporal_load(reinterpret_cast<const Raw*>(p)));
}
template <class P>
__device__ __forceinline__ void store_stream(void* p, const P& x) {
    typedef typename RawBits<sizeof(P)>::type Raw;
    __builtin_nontemporal_store(__builtin_bit_cast(Raw, x), reinterpret_cast<Raw*>(p));
}

// Persistent blocks: block b moves tiles b, b + gridDim.x, ...  The next tile's global loads are issued
// (into registers) before the current tile is written out, so loads stay in flight during the store phase.
// VR / VW: elements per global access on the read / write side (16-byte accesses when the layout allows).
// Interior tiles take a fast path: the in-tile byte offsets and LDS positions of each thread's accesses are
// computed once (32-bit) and reused for every tile against a uniform per-tile base; edge tiles and tensors
// whose tiles span 4 GiB recompute coordinates with bounds checks.
// FULL (with FAST): the tile has exactly EPT * NTH elements, so no access is masked and the tile loop is straight-line
// code.  With per-access masks every load sits in its own conditional block; the compiler then cannot tell that the
// previous tile's loads have completed and makes each load of the next tile wait for the one before it.
template <class V, class Op, int EPT, int VR, int VW, bool READ_OLD, bool FAST, int NTH = THREADS, bool FULL = false>
__global__ void __launch_bounds__(NTH) copy_kernel(CopyArgs a, Op op) {
    prefetch_kernel_arguments<sizeof(CopyArgs)>();
    extern __shared__ __align__(16) unsigned char smem_raw[];
    V* lds = reinterpret_cast<V*>(smem_raw);
    constexpr int NR = EPT / VR, NW = EPT / VW;
    int tid = threadIdx.x;
    V regs[EPT];
    uint32_t roff[FAST ? NR : 1], woff[FAST ? NW : 1];
    int wl[FAST ? NW : 1];
    uint32_t rmask = 0, wmask = 0;
    if constexpr (FULL) {
        static_assert(NR <= MAXU && NW <= MAXU, "the host provides MAXU per-access offsets");
        // tile coordinates are bit fields of the tile position, and the position splits into disjoint bits from the
        // thread and from u: offsets are sums of a per-thread part (here) and a per-u part (from the host)
        const int r0 = tid * VR;
        uint32_t mine = 0u - a.in_rebase_b;
#pragma unroll
        for (int t = 0; t < MAXT; ++t) mine += (uint32_t)((r0 >> a.r_shift[t]) & a.r_mask[t]) * a.r_sb[t];
#pragma clang loop unroll(full)
        for (int u = 0; u < NR; ++u) roff[u] = mine + a.u_roff[u];
    } else {
#pragma clang loop unroll(full)
    for (int u = 0; u < (FAST ? NR : 0); ++u) {
        const int r = (u * NTH + tid) * VR;
        int64_t off = 0;
#pragma unroll
        for (int t = 0; t < MAXT; ++t) off += (int64_t)((r >> a.r_shift[t]) & a.r_mask[t]) * a.r_si[t];
        roff[u] = (uint32_t)((off - a.in_rebase) * (int64_t)sizeof(V));
        rmask |= (r < a.tile_elems ? 1u : 0u) << u;
    }
    }
    if constexpr (FULL) {
        const int w0 = tid * VW;
        uint32_t mine = 0u - a.out_rebase_b;
        int r = 0;
#pragma unroll
        for (int t = 0; t < MAXT; ++t) {
            const int c = (w0 >> a.w_shift[t]) & a.w_mask[t];
            mine += (uint32_t)c * a.w_sb[t];
            r += c * a.w_rpos[t];
        }
#pragma clang loop unroll(full)
        for (int u = 0; u < NW; ++u) {
            woff[u] = mine + a.u_woff[u];
            wl[u] = r + a.u_wl[u];
        }
    } else {
#pragma clang loop unroll(full)
        for (int u = 0; u < (FAST ? NW : 0); ++u) {
            const int w = (u * NTH + tid) * VW;
            int64_t off = 0;
            int r = 0;
#pragma unroll
            for (int t = 0; t < MAXT; ++t) {
                const int c = (w >> a.w_shift[t]) & a.w_mask[t];
                off += (int64_t)c * a.w_so[t];
                r += c * a.w_rpos[t];
            }
            woff[u] = (uint32_t)((off - a.out_rebase) * (int64_t)sizeof(V));
            wl[u] = r;
            wmask |= (w < a.tile_elems ? 1u : 0u) << u;
        }
    }

    auto load = [&](const BlockOrigin& o) {
        if constexpr (FAST) {
            // the complete tile base goes through readfirstlane: an opaque scalar that the optimiser cannot split up again
            // (it otherwise hoists "input pointer + thread offset" out of the tile loop as 64-bit vector addresses, adds the
            // tile origin to each on the vector unit, and lets those address registers share the loads' destinations, so
            // that every load of the next tile waits for the previous one)
            const gcptr base = (gcptr)(uintptr_t)uniform64((int64_t)(uintptr_t)(reinterpret_cast<const V*>(a.in) + o.in + a.in_rebase));
#pragma clang loop unroll(full)
            for (int u = 0; u < NR; ++u) {
                if (FULL || ((rmask >> u) & 1u)) {
                    const Pack<V, VR> p = gload_pack<Pack<V, VR>>(base, roff[u]);
#pragma unroll
                    for (int j = 0; j < VR; ++j) regs[u * VR + j] = p.v[j];
                }
            }
            return;
        } else {
        // hide the tile-invariance of this index arithmetic so that it is not hoisted into ~100 registers
        asm volatile("" : "+v"(tid));
        const V* in = reinterpret_cast<const V*>(a.in) + o.in;
#pragma clang loop unroll(full)
        for (int u = 0; u < NR; ++u) {
            const int r = (u * NTH + tid) * VR;
            bool ok = r < a.tile_elems;
            int64_t off = 0;
#pragma unroll
            for (int t = 0; t < MAXT; ++t) {   // unused axis slots are neutral: mask 0, stride 0, id 0
                const int c = (r >> a.r_shift[t]) & a.r_mask[t];
                off += (int64_t)c * a.r_si[t];
                ok &= c < pick_lim(o, a.r_id[t]);
            }
            if (ok) {
                const Pack<V, VR> p = load_stream<Pack<V, VR>>(in + off);
#pragma unroll
                for (int j = 0; j < VR; ++j) regs[u * VR + j] = p.v[j];
            }
        }
        }
    };
    uint64_t tile = blockIdx.x;
    if (tile >= (uint64_t)a.ntiles) return;
    BlockOrigin o;
    o.in = o.in2 = o.out = 0;
#pragma unroll
    for (int t = 0; t < MAXT; ++t) o.lim[t] = 0;   // (the straight-line variant never looks at lim)
    TileWalk walk;
    if constexpr (FULL) {
        walk.start(a, (uint32_t)tile);
        walk.offsets(a, o.in, o.out);
    } else {
        o = block_origin(a, tile);
    }
    load(o);
    // (nothing that the tile loop needs later -- LDS positions, write offsets -- is to be computed ahead of these loads)
    if constexpr (FULL) __builtin_amdgcn_sched_barrier(0);
    for (;;) {
#pragma clang loop unroll(full)
        for (int u = 0; u < NR; ++u) {
            const int r = (u * NTH + tid) * VR;
            if (FULL || (FAST ? (bool)((rmask >> u) & 1u) : r < a.tile_elems)) {
#pragma unroll
                for (int j = 0; j < VR; ++j) lds[swz(r) + j] = regs[u * VR + j];
            }
        }
        __syncthreads();
        const uint64_t next = tile + gridDim.x;
        const bool more = next < (uint64_t)a.ntiles;
        BlockOrigin o2 = o;
        if (more) {
            if constexpr (FULL) {
                walk.advance(a);
                walk.offsets(a, o2.in, o2.out);
            } else {
                o2 = block_origin(a, next);
            }
            load(o2);
        }
        if constexpr (FAST) {
            const gmptr base = (gmptr)(uintptr_t)uniform64((int64_t)(uintptr_t)(reinterpret_cast<V*>(a.out) + o.out + a.out_rebase));
#pragma clang loop unroll(full)
            for (int u = 0; u < NW; ++u) {
                if (FULL || ((wmask >> u) & 1u)) {
                    Pack<V, VW> x, old;
#pragma unroll
                    for (int j = 0; j < VW; ++j) x.v[j] = lds[swz(wl[u] + j * a.w_rpos[0])];
                    old = x;
                    if (READ_OLD) old = gload_pack<Pack<V, VW>>((gcptr)base, woff[u]);
#pragma unroll
                    for (int j = 0; j < VW; ++j) x.v[j] = op(x.v[j], old.v[j], a);
                    gstore_pack<Pack<V, VW>>(base, woff[u], x);
                }
            }
        } else {
            V* out = reinterpret_cast<V*>(a.out) + o.out;
            asm volatile("" : "+v"(tid));
#pragma clang loop unroll(full)
            for (int u = 0; u < NW; ++u) {
                const int w = (u * NTH + tid) * VW;
                bool ok = w < a.tile_elems;
                int64_t off = 0;
                int r = 0;
#pragma unroll
                for (int t = 0; t < MAXT; ++t) {
                    const int c = (w >> a.w_shift[t]) & a.w_mask[t];
                    off += (int64_t)c * a.w_so[t];
                    r += c * a.w_rpos[t];
                    ok &= c < pick_lim(o, a.w_id[t]);
                }
                if (ok) {
                    Pack<V, VW> x, old;
#pragma unroll
                    for (int j = 0; j < VW; ++j) x.v[j] = lds[swz(r + j * a.w_rpos[0])];
                    old = x;
                    if (READ_OLD) old = load_stream<Pack<V, VW>>(out + off);
#pragma unroll
                    for (int j = 0; j < VW; ++j) x.v[j] = op(x.v[j], old.v[j], a);
                    store_stream<Pack<V, VW>>(out + off, x);
                }
            }
        }
        if (!more) break;
        __syncthreads();
        tile = next;
        o = o2;
    }
}

// ---- tiles of many short axes ---------------------------------------------------------------------------------------
// A tensor of many small extents (3^14, 2^16, [3,4]x6: spins and qubits) has no long axis to tile: four power-of-two tile
// axes give runs of a few elements and, for extents that are no powers of two, mostly idle lanes (3^14 reversed:
// 161 GB/s).  Here a tile is the product of whole axes -- as many as it takes to reach 512-byte runs on both sides --
// and, where a whole axis does not fit, of a range of its indices (one such axis per side at most: a long extent that
// is no power of two, [27,466,1401]), and the position-to-offset maps of a tile, which no longer are shifts and masks,
// come from tables built once per layout (input offset in read order; output offset and LDS position in write order)
// and kept in registers for all the tiles a block moves.  Only the last range of a ranged axis is ragged: a tile
// there looks up the coordinates of its positions along the ranged axes in two more tables and leaves out what lies
// past the edge; every other tile is full.
constexpr int TAB_MAX_AXES = 16;
struct TabCopyArgs {
    const void* in;
    void* out;
    // [5][E]: input element offset of read position r; output offset and LDS position of write position w; the
    // coordinates along the two ranged axes (16 bits each) of read position r, and of write position w
    const uint32_t* tab;
    int32_t E, ng;
    int64_t ntiles;
    int64_t g_count[MAXG], g_si[MAXG], g_so[MAXG];
    int32_t g_slot[MAXG];    // 1, 2: the tile index along ranged axis 1, 2; 0: an axis outside the tile
    int32_t x_n[2], x_t[2];  // extent of a ranged axis and its indices per tile (1, 1 when there is none)
};
struct TabBuildArgs {
    uint32_t* tab;
    int32_t E, nt;
    int32_t r_ext[TAB_MAX_AXES], w_ext[TAB_MAX_AXES], w_rpos[TAB_MAX_AXES];
    int32_t r_slot[TAB_MAX_AXES], w_slot[TAB_MAX_AXES];   // 1, 2: a ranged axis; 0: a whole one
    int64_t r_si[TAB_MAX_AXES], w_so[TAB_MAX_AXES];
};
__global__ void __launch_bounds__(THREADS) tabcopy_build_kernel(TabBuildArgs b) {
    const int i = blockIdx.x * THREADS + threadIdx.x;
    if (i >= b.E) return;
    int lin = i;
    int64_t off = 0;
    uint32_t xc = 0;
    for (int t = 0; t < b.nt; ++t) {
        const int q = lin / b.r_ext[t], c = lin - q * b.r_ext[t];
        off += (int64_t)c * b.r_si[t];
        if (b.r_slot[t]) xc |= (uint32_t)c << (16 * (b.r_slot[t] - 1));
        lin = q;
    }
    b.tab[i] = (uint32_t)off;
    b.tab[3 * b.E + i] = xc;
    lin = i;
    off = 0;
    xc = 0;
    int pos = 0;
    for (int t = 0; t < b.nt; ++t) {
        const int q = lin / b.w_ext[t], c = lin - q * b.w_ext[t];
        off += (int64_t)c * b.w_so[t];
        pos += c * b.w_rpos[t];
        if (b.w_slot[t]) xc |= (uint32_t)c << (16 * (b.w_slot[t] - 1));
        lin = q;
    }
    b.tab[b.E + i] = (uint32_t)off;
    b.tab[2 * b.E + i] = (uint32_t)pos;
    b.tab[4 * b.E + i] = xc;
}

// Tile t of a block on XCD x (blocks go to the XCDs in turn) -> a tile index such that every XCD moves one contiguous
// eighth of the tiles: tiles that abut in memory share 128-byte lines at their edges, and meet in one L2.
__device__ __forceinline__ uint64_t tab_tile_of(uint64_t slot, uint64_t ntiles) {
    const uint64_t per = (ntiles + 7) / 8;
    return (slot & 7) * per + (slot >> 3);
}

template <class V, int EPT>
__global__ void __launch_bounds__(THREADS) tabcopy_kernel(TabCopyArgs a) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    V* lds = reinterpret_cast<V*>(smem_raw);
    const int tid = threadIdx.x, E = a.E;
    uint32_t roff[EPT], woff[EPT], lpos[EPT];
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
        const int r = tid + THREADS * j;
        roff[j] = woff[j] = lpos[j] = 0;
        if (r < E) {
            roff[j] = a.tab[r];
            woff[j] = a.tab[E + r];
            lpos[j] = swz((int)a.tab[2 * E + r]);
        }
    }
    // origin of a tile and the indices of the ranged axes it holds, packed like the coordinates in the tables
    auto origin = [&](uint64_t tile, int64_t& oi, int64_t& oo, uint32_t& lim) {
        oi = oo = 0;
        int l[2] = {a.x_t[0], a.x_t[1]};
        for (int g = 0; g < a.ng; ++g) {
            const uint64_t q = tile / (uint64_t)a.g_count[g];
            const int64_t c = (int64_t)(tile - q * (uint64_t)a.g_count[g]);
            tile = q;
            oi += c * a.g_si[g];
            oo += c * a.g_so[g];
#pragma unroll
            for (int x = 0; x < 2; ++x)
                if (a.g_slot[g] == x + 1) {
                    const int64_t left = (int64_t)a.x_n[x] - c * a.x_t[x];
                    if (left < l[x]) l[x] = (int)left;
                }
        }
        oi = uniform64(oi);
        oo = uniform64(oo);
        lim = (uint32_t)__builtin_amdgcn_readfirstlane(l[0] | (l[1] << 16));
    };
    const uint32_t lim_full = (uint32_t)(a.x_t[0] | (a.x_t[1] << 16));
    auto inside = [&](uint32_t xc, uint32_t lim) { return (xc & 0xffffu) < (lim & 0xffffu) && (xc >> 16) < (lim >> 16); };
    V regs[EPT];
    auto load = [&](int64_t oi, uint32_t lim) {
        const V* in = reinterpret_cast<const V*>(a.in) + oi;
        if (lim == lim_full) {
#pragma unroll
            for (int j = 0; j < EPT; ++j)
                if (tid + THREADS * j < E) regs[j] = load_stream<Pack<V, 1>>(in + roff[j]).v[0];
        } else {   // a tile at a ragged edge: the positions past the edge are left out
#pragma unroll
            for (int j = 0; j < EPT; ++j) {
                const int r = tid + THREADS * j;
                if (r < E && inside(a.tab[3 * E + r], lim)) regs[j] = load_stream<Pack<V, 1>>(in + roff[j]).v[0];
            }
        }
    };
    const uint64_t ntiles = (uint64_t)a.ntiles, slots = (ntiles + 7) / 8 * 8;
    uint64_t slot = blockIdx.x;
    while (slot < slots && tab_tile_of(slot, ntiles) >= ntiles) slot += gridDim.x;
    if (slot >= slots) return;
    int64_t oi, oo;
    uint32_t lim;
    origin(tab_tile_of(slot, ntiles), oi, oo, lim);
    load(oi, lim);
    for (;;) {
#pragma unroll
        for (int j = 0; j < EPT; ++j) {
            const int r = tid + THREADS * j;
            if (r < E) lds[swz(r)] = regs[j];
        }
        __syncthreads();
        uint64_t next = slot + gridDim.x;
        while (next < slots && tab_tile_of(next, ntiles) >= ntiles) next += gridDim.x;
        const bool more = next < slots;
        int64_t oi2 = 0, oo2 = 0;
        uint32_t lim2 = lim_full;
        if (more) {   // the next tile's loads are in flight while this one is written out
            origin(tab_tile_of(next, ntiles), oi2, oo2, lim2);
            load(oi2, lim2);
        }
        V* out = reinterpret_cast<V*>(a.out) + oo;
        if (lim == lim_full) {
#pragma unroll
            for (int j = 0; j < EPT; ++j)
                if (tid + THREADS * j < E) {
                    Pack<V, 1> x;
                    x.v[0] = lds[lpos[j]];
                    out[woff[j]] = x.v[0];   // (a cached store: runs start anywhere, and neighbours complete the lines they share)
                }
        } else {
#pragma unroll
            for (int j = 0; j < EPT; ++j) {
                const int w = tid + THREADS * j;
                if (w < E && inside(a.tab[4 * E + w], lim)) {
                    Pack<V, 1> x;
                    x.v[0] = lds[lpos[j]];
                    out[woff[j]] = x.v[0];   // (a cached store: runs start anywhere, and neighbours complete the lines they share)
                }
            }
        }
        if (!more) break;
        __syncthreads();
        slot = next;
        oo = oo2;
        lim = lim2;
    }
}

// Direct (no LDS) kernels in write order: fill and elementwise multiply.
template <class V>
__global__ void __launch_bounds__(THREADS) fill_kernel(CopyArgs a, V value, int ept) {
    const BlockOrigin o = block_origin(a, (uint64_t)blockIdx.x + (uint64_t)blockIdx.y * gridDim.x);
    V* out = reinterpret_cast<V*>(a.out) + o.out;
    for (int u = 0; u < ept; ++u) {
        int w = u * THREADS + threadIdx.x;
        bool ok = w < a.tile_elems;
        int64_t off = 0;
        for (int t = 0; t < a.nt; ++t) {
            int c = (w >> a.w_shift[t]) & a.w_mask[t];
            off += (int64_t)c * a.w_so[t];
            ok &= c < pick_lim(o, a.w_id[t]);
        }
        if (ok) out[off] = value;
    }
}

template <class R, bool CX>
__global__ void __launch_bounds__(THREADS) emul_kernel(CopyArgs a, int ept) {
    prefetch_kernel_arguments<sizeof(CopyArgs)>();
    constexpr int NC = CX ? 2 : 1;
    const BlockOrigin o = block_origin(a, (uint64_t)blockIdx.x + (uint64_t)blockIdx.y * gridDim.x);
    const R* A = reinterpret_cast<const R*>(a.in) + o.in * NC;
    const R* B = reinterpret_cast<const R*>(a.in2) + o.in2 * NC;
    R* C = reinterpret_cast<R*>(a.out) + o.out * NC;
    for (int u = 0; u < ept; ++u) {
        int w = u * THREADS + threadIdx.x;
        bool ok = w < a.tile_elems;
        int64_t oa = 0, ob = 0, oc = 0;
        for (int t = 0; t < a.nt; ++t) {
            int c = (w >> a.w_shift[t]) & a.w_mask[t];
            oa += (int64_t)c * a.w_si[t];
            ob += (int64_t)c * a.w_si2[t];
            oc += (int64_t)c * a.w_so[t];
            ok &= c < pick_lim(o, a.w_id[t]);
        }
        if (!ok) continue;
        R ar = (R)a.alpha_re, ai = (R)a.alpha_im;
        if (CX) {
            R xr = A[oa * 2], xi = A[oa * 2 + 1], yr = B[ob * 2], yi = B[ob * 2 + 1];
            R pr = xr * yr - xi * yi, pi = xr * yi + xi * yr;
            R rr = ar * pr - ai * pi, ri = ar * pi + ai * pr;
            if (a.use_beta) {
                R br = (R)a.beta_re, bi = (R)a.beta_im, cr = C[oc * 2], ci = C[oc * 2 + 1];
                rr += br * cr - bi * ci;
                ri += br * ci + bi * cr;
            }
            C[oc * 2] = rr;
            C[oc * 2 + 1] = ri;
        } else {
            R r = ar * (A[oa] * B[ob]);
            if (a.use_beta) r += (R)a.beta_re * C[oc];
            C[oc] = r;
        }
    }
}

// ---- host side: tile selection --------------------------------------------------------------------------
int ceil_log2(int64_t n) {
    int l = 0;
    while (((int64_t)1 << l) < n) ++l;
    return l;
}

struct TilePlan {
    CopyArgs args;
    dim3 grid;
    int ept;
    bool vec_in, vec_out;   // strides allow 16-byte accesses on the input / output side
    bool all_full;          // no partial tiles and 32-bit in-tile offsets: the kernel's fast path applies
    uint32_t persistent;    // block count for the looping copy kernel
};

// axes: s[0] = input stride, s[1] = output stride, s[2] = second input stride (emul only).
// order_slot: which slot defines the read order (0) -- the write order is always slot 1.
// grow_side / grow_log2: after the tile is chosen within max_tile_elems, the run of one side (0 = input, 1 = output) is
// lengthened by up to grow_log2 more doublings (the large-tile variant of the copy kernel).
int32_t plan_tiles(std::vector<Axis> axes, int elem_bytes, int max_tile_elems, bool two_sided, TilePlan& tp, int grow_side = -1,
                   int grow_log2 = 0) {
    CopyArgs& a = tp.args;
    std::memset(&a, 0, sizeof a);
    for (auto& x : axes)
        if (x.n == 0) {
            tp.grid = dim3(0, 0, 0);
            return TFH_OK;
        }
    // canonical order: output stride descending, then merge what is contiguous on every side
    std::stable_sort(axes.begin(), axes.end(), [](const Axis& x, const Axis& y) { return std::llabs(x.s[1]) > std::llabs(y.s[1]); });
    fuse_axes(axes, 3);
    if (axes.empty()) axes.push_back(Axis{1, {0, 0, 0}, 0});
    const int na = (int)axes.size();
    if (na > MAXG) return set_error(TFH_ERR_INVALID_ARGUMENT, "more than %d non-mergeable axes", MAXG);
    for (auto& x : axes)
        if (x.n > 1 && x.s[1] == 0) return set_error(TFH_ERR_STRIDED, "output view has stride 0 on an axis of extent %lld (elements would alias)", (long long)x.n);
    auto key_in = [&](int i) { return axes[i].s[0] == 0 ? INT64_MAX : std::llabs(axes[i].s[0]); };
    std::vector<int> out_order(na), in_order(na);
    for (int i = 0; i < na; ++i) out_order[i] = in_order[i] = i;
    std::stable_sort(out_order.begin(), out_order.end(), [&](int x, int y) { return std::llabs(axes[x].s[1]) < std::llabs(axes[y].s[1]); });
    std::stable_sort(in_order.begin(), in_order.end(), [&](int x, int y) { return key_in(x) < key_in(y); });

    std::vector<int> tl(na, 0);  // log2 tile extent per axis
    // An extent that is not a power of two makes its last tile partial, and one partial tile takes the whole launch
    // off the kernel's fast path.  When the extent has a power-of-two divisor of at least 128 bytes (96 = 3 x 32), the
    // tile is first tried no longer than that divisor; the plan is kept if every tile then comes out full.
    bool capped = false;
    auto full = [&](int i) {
        const int64_t n = axes[i].n;
        const int whole = ceil_log2(n);
        if (!capped || (n & (n - 1)) == 0) return whole;
        const int d = __builtin_ctzll((unsigned long long)n);
        return ((int64_t)elem_bytes << d) >= 128 ? d : whole;
    };
    auto tile_axes = [&]() { int c = 0; for (int i = 0; i < na; ++i) c += tl[i] > 0; return c; };
    auto prod_log2 = [&]() { int p = 0; for (int i = 0; i < na; ++i) p += tl[i]; return p; };
    const int budget = ceil_log2(max_tile_elems);
    const int run_target = ceil_log2(std::max(1, 512 / elem_bytes));
    auto take_run = [&](const std::vector<int>& order) {
        int run = 0;
        for (int i : order) {
            if (run >= run_target) break;
            if (tl[i] == 0 && tile_axes() >= MAXT) break;
            int want = std::min(full(i), run_target - run);
            want = std::max(want, tl[i]);
            want = std::min(want, tl[i] + budget - prod_log2());
            tl[i] = want;
            run += want;
            if (want < ceil_log2(axes[i].n)) break;   // the run ends at an axis the tile covers only partly
        }
    };
    auto choose = [&]() {
        std::fill(tl.begin(), tl.end(), 0);
        take_run(out_order);
        if (two_sided) take_run(in_order);
        // spend the rest of the budget: alternately lengthen the output-side and the input-side run
        for (int side = 0; prod_log2() < budget; side ^= 1) {
            bool grew = false;
            for (int pass = 0; pass < 2 && !grew; ++pass) {
                const std::vector<int>& order = ((side ^ pass) == 0 || !two_sided) ? out_order : in_order;
                for (int i : order) {
                    if (tl[i] < full(i) && (tl[i] > 0 || tile_axes() < MAXT)) {
                        ++tl[i];
                        grew = true;
                        break;
                    }
                    if (tl[i] < ceil_log2(axes[i].n)) break;  // cannot extend this run past a partial axis
                }
            }
            if (!grew) break;
        }
        if (grow_side >= 0) {
            const std::vector<int>& order = grow_side == 1 ? out_order : in_order;
            for (int more = 0; more < grow_log2; ++more) {
                bool grew = false;
                for (int i : order) {
                    if (tl[i] < full(i) && (tl[i] > 0 || tile_axes() < MAXT)) {
                        ++tl[i];
                        grew = true;
                        break;
                    }
                    if (tl[i] < ceil_log2(axes[i].n)) break;
                }
                if (!grew) break;
            }
        }
    };
    for (int i = 0; i < na; ++i) capped = capped || (axes[i].n & (axes[i].n - 1)) != 0;
    if (capped) {
        choose();
        bool all_full = true;
        for (int i = 0; i < na; ++i) all_full = all_full && (tl[i] == 0 || axes[i].n % ((int64_t)1 << tl[i]) == 0);
        const std::vector<int> tl_capped = tl;
        const int elems_capped = prod_log2();
        capped = false;
        choose();
        // (a capped plan whose tile came out tiny would trade the fast path for too little work per block)
        if (all_full && (elems_capped >= 10 || elems_capped + 1 >= prod_log2())) tl = tl_capped;
    } else {
        choose();
    }
    // tile axis ids
    std::vector<int> ids;
    for (int i = 0; i < na; ++i)
        if (tl[i] > 0) ids.push_back(i);
    a.nt = (int)ids.size();
    a.tile_elems = 1 << prod_log2();
    auto id_of = [&](int axis) { return (int)(std::find(ids.begin(), ids.end(), axis) - ids.begin()); };
    for (int t = 0; t < a.nt; ++t) a.t_n[t] = axes[ids[t]].n;
    // read order / write order
    std::vector<int> rd, wr;
    for (int i : in_order) if (tl[i] > 0) rd.push_back(i);
    for (int i : out_order) if (tl[i] > 0) wr.push_back(i);
    std::vector<int> rshift(na, 0);
    int sh = 0;
    for (int t = 0; t < a.nt; ++t) {
        int i = rd[t];
        a.r_shift[t] = sh;
        a.r_mask[t] = (1 << tl[i]) - 1;
        a.r_id[t] = id_of(i);
        a.r_si[t] = axes[i].s[0];
        rshift[i] = sh;
        sh += tl[i];
    }
    sh = 0;
    for (int t = 0; t < a.nt; ++t) {
        int i = wr[t];
        a.w_shift[t] = sh;
        a.w_mask[t] = (1 << tl[i]) - 1;
        a.w_id[t] = id_of(i);
        a.w_rpos[t] = 1 << rshift[i];
        a.w_so[t] = axes[i].s[1];
        a.w_si[t] = axes[i].s[0];
        a.w_si2[t] = axes[i].s[2];
        sh += tl[i];
    }
    // fast path data: tile extents and the lowest in-tile offset per side; usable when the tile spans < 4 GiB
    {
        int64_t lo_in = 0, hi_in = 0, lo_out = 0, hi_out = 0;
        for (int t = 0; t < MAXT; ++t) a.t_text[t] = 1;
        for (int t = 0; t < a.nt; ++t) {
            const int i = ids[t];
            const int64_t ext = ((int64_t)1 << tl[i]) - 1;
            a.t_text[t] = 1 << tl[i];
            (axes[i].s[0] < 0 ? lo_in : hi_in) += ext * axes[i].s[0];
            (axes[i].s[1] < 0 ? lo_out : hi_out) += ext * axes[i].s[1];
        }
        a.in_rebase = lo_in;
        a.out_rebase = lo_out;
        a.fast32 = (hi_in - lo_in + 1) * (int64_t)elem_bytes < ((int64_t)1 << 32) &&
                   (hi_out - lo_out + 1) * (int64_t)elem_bytes < ((int64_t)1 << 32);
        tp.all_full = a.fast32 != 0;
        for (int t = 0; t < a.nt; ++t) tp.all_full &= axes[ids[t]].n % ((int64_t)1 << tl[ids[t]]) == 0;
    }
    // grid axes; the axes a tile covers only partly come first (fastest block index), so blocks that run at
    // the same time complete each other's contiguous runs in DRAM
    a.ng = 0;
    uint64_t blocks = 1;
    for (int pass = 0; pass < 2; ++pass)
        for (int i = 0; i < na; ++i) {
            int64_t text = (int64_t)1 << tl[i];
            int64_t cnt = (axes[i].n + text - 1) / text;
            if (cnt <= 1) continue;
            if ((pass == 0) != (tl[i] > 0)) continue;
            int g = a.ng++;
            a.g_count[g] = cnt;
            a.g_si[g] = axes[i].s[0] * text;
            a.g_si2[g] = axes[i].s[2] * text;
            a.g_so[g] = axes[i].s[1] * text;
            a.g_tid[g] = tl[i] > 0 ? id_of(i) : -1;
            a.g_text[g] = (int32_t)text;
            blocks *= (uint64_t)cnt;
        }
    for (int g = a.ng; g < MAXG; ++g) a.g_count[g] = 1;   // neutral: the kernels' unconditional tile walk relies on it
    a.ntiles = (int64_t)blocks;
    // 4 resident blocks per CU on 256 CUs; block counts from 512 to 4096 measure within 2% of each other
    tp.persistent = (uint32_t)std::min<uint64_t>(blocks, 1024);
    // 16-byte accesses: the side's fastest tile axis is contiguous, a multiple of the vector length, and every
    // other stride keeps the vectors aligned
    const int vec = 16 / elem_bytes;
    auto side_ok = [&](int slot, const std::vector<int>& order_) {
        if (vec <= 1 || order_.empty()) return false;
        const int i0 = order_[0];
        if (axes[i0].s[slot] != 1 || axes[i0].n % vec != 0 || (1 << tl[i0]) < vec) return false;
        for (int i = 0; i < na; ++i)
            if (i != i0 && axes[i].s[slot] % vec != 0) return false;
        return true;
    };
    tp.vec_in = side_ok(0, rd);
    tp.vec_out = side_ok(1, wr);
    if (blocks > (uint64_t)0x7fffffff * 65535ull) return set_error(TFH_ERR_INVALID_ARGUMENT, "tensor too large for one launch");
    uint32_t gx = (uint32_t)std::min<uint64_t>(blocks, 0x7fffffffull);
    uint32_t gy = (uint32_t)((blocks + gx - 1) / gx);
    if ((uint64_t)gx * gy != blocks) {  // keep the grid exact: x*y must equal the block count
        gx = 1u << 30;
        while (blocks % gx) gx >>= 1;
        gy = (uint32_t)(blocks / gx);
        if (gy > 65535u) return set_error(TFH_ERR_INVALID_ARGUMENT, "tensor too large for one launch");
    }
    tp.grid = dim3(gx, gy, 1);
    tp.ept = (a.tile_elems + THREADS - 1) / THREADS;
    return TFH_OK;
}

void set_scalars(CopyArgs& a, Scalar alpha, Scalar beta, bool conj) {
    a.alpha_re = alpha.re;
    a.alpha_im = alpha.im;
    a.beta_re = beta.re;
    a.beta_im = beta.im;
    a.conj = conj;
    a.use_beta = !beta.is_zero();
}

// Large tiles (raw moves only): 512 threads move a tile of 32 elements per thread (128 KB of 8-byte elements), one block
// per CU.  Every tile is full and both sides take 16-byte accesses.
template <class V, int EPT>
void launch_copy_large(TilePlan& tp, size_t lds, hipStream_t st) {
    constexpr int VEC = 16 / sizeof(V);
    {   // the per-u parts of the offsets (see CopyArgs)
        CopyArgs& a = tp.args;
        uint32_t step = tp.persistent;
        for (int g = 0; g < WALKG; ++g) {
            a.walk_inc[g] = step % (uint32_t)a.g_count[g];
            step /= (uint32_t)a.g_count[g];
            a.walk_magic[g] = a.g_count[g] <= 1 ? 0xffffffffu : (uint32_t)(((uint64_t)1 << 32) / (uint64_t)a.g_count[g]);
        }
        for (int t = 0; t < MAXT; ++t) {
            a.r_sb[t] = (uint32_t)(a.r_si[t] * (int64_t)sizeof(V));
            a.w_sb[t] = (uint32_t)(a.w_so[t] * (int64_t)sizeof(V));
        }
        a.in_rebase_b = (uint32_t)(a.in_rebase * (int64_t)sizeof(V));
        a.out_rebase_b = (uint32_t)(a.out_rebase * (int64_t)sizeof(V));
        for (int u = 0; u < EPT / VEC; ++u) {
            const int pos = u * 512 * VEC;
            int64_t offr = 0, offw = 0;
            int rp = 0;
            for (int t = 0; t < MAXT; ++t) {
                offr += (int64_t)((pos >> a.r_shift[t]) & a.r_mask[t]) * a.r_si[t];
                const int c = (pos >> a.w_shift[t]) & a.w_mask[t];
                offw += (int64_t)c * a.w_so[t];
                rp += c * a.w_rpos[t];
            }
            a.u_roff[u] = (uint32_t)(offr * (int64_t)sizeof(V));
            a.u_woff[u] = (uint32_t)(offw * (int64_t)sizeof(V));
            a.u_wl[u] = rp;
        }
    }
    static bool once = [] {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&copy_kernel<V, RawOp<V>, EPT, VEC, VEC, false, true, 512, true>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        return true;
    }();
    (void)once;
    TFH_LAUNCH_TIMED((copy_kernel<V, RawOp<V>, EPT, VEC, VEC, false, true, 512, true>), dim3(tp.persistent), dim3(512), lds, st, tp.args, RawOp<V>());
}

template <class V, class Op, int EPT, int VR, int VW>
void launch_copy_variant(const TilePlan& tp, Op op, bool read_old, size_t lds, hipStream_t st) {
    const dim3 grid(tp.persistent), block(THREADS);
    // FAST: every tile is full (each tiled extent is a multiple of its tile extent) and spans < 4 GiB
    if (tp.all_full) {
        if (read_old) TFH_LAUNCH_TIMED((copy_kernel<V, Op, EPT, VR, VW, true, true>), grid, block, lds, st, tp.args, op);
        else TFH_LAUNCH_TIMED((copy_kernel<V, Op, EPT, VR, VW, false, true>), grid, block, lds, st, tp.args, op);
    } else {
        if (read_old) TFH_LAUNCH_TIMED((copy_kernel<V, Op, EPT, VR, VW, true, false>), grid, block, lds, st, tp.args, op);
        else TFH_LAUNCH_TIMED((copy_kernel<V, Op, EPT, VR, VW, false, false>), grid, block, lds, st, tp.args, op);
    }
}

// ALLVEC: also instantiate the mixed (vector on one side only) variants.
template <class V, class Op, bool ALLVEC>
int32_t run_copy(const TilePlan& tp, Op op, bool read_old, bool vin, bool vout, hipStream_t st) {
    constexpr int VEC = 16 / sizeof(V);
    constexpr int BIG = sizeof(V) >= 16 ? 8 : 16;
    const size_t lds = (size_t)(tp.args.tile_elems + tp.args.tile_elems / 32 + 4) * sizeof(V);
    const int prof = prof_begin(PROF_COPY, st);
    const bool big = tp.ept > 4;
    if constexpr (VEC == 1) {
        if (big) launch_copy_variant<V, Op, BIG, 1, 1>(tp, op, read_old, lds, st);
        else launch_copy_variant<V, Op, 4, 1, 1>(tp, op, read_old, lds, st);
    } else {
        if (!ALLVEC && !(vin && vout)) vin = vout = false;
        if (big) {
            if (vin && vout) launch_copy_variant<V, Op, BIG, VEC, VEC>(tp, op, read_old, lds, st);
            else if constexpr (ALLVEC) {
                if (vin) launch_copy_variant<V, Op, BIG, VEC, 1>(tp, op, read_old, lds, st);
                else if (vout) launch_copy_variant<V, Op, BIG, 1, VEC>(tp, op, read_old, lds, st);
                else launch_copy_variant<V, Op, BIG, 1, 1>(tp, op, read_old, lds, st);
            } else launch_copy_variant<V, Op, BIG, 1, 1>(tp, op, read_old, lds, st);
        } else {
            if (vin && vout && tp.args.tile_elems >= THREADS * VEC) launch_copy_variant<V, Op, 4, VEC, VEC>(tp, op, read_old, lds, st);
            else launch_copy_variant<V, Op, 4, 1, 1>(tp, op, read_old, lds, st);
        }
    }
    prof_end(prof, st);
    return hip_check(hipGetLastError(), "copy kernel launch");
}

bool aligned(const void* p, size_t a) { return ((uintptr_t)p % a) == 0; }

}  // namespace

namespace {
// Contiguous run (elements) a tile of the shift-and-mask plan reads (slot 0) or writes (slot 1), and the share of its
// positions that hold an element (tile extents are powers of two, the axes need not be).
void masked_plan_quality(const CopyArgs& a, int64_t& run_in, int64_t& run_out, double& filled) {
    run_in = run_out = 1;
    filled = 1.0;
    bool go = true;
    for (int t = 0; t < a.nt && go; ++t) {
        const int64_t ext = a.r_mask[t] + 1, n = a.t_n[a.r_id[t]], use = std::min(ext, n);
        if (std::llabs(a.r_si[t]) != run_in) break;
        run_in *= use;
        go = use == n;
    }
    go = true;
    for (int t = 0; t < a.nt && go; ++t) {
        const int64_t ext = a.w_mask[t] + 1, n = a.t_n[a.w_id[t]], use = std::min(ext, n);
        if (std::llabs(a.w_so[t]) != run_out) break;
        run_out *= use;
        go = use == n;
    }
    for (int t = 0; t < a.nt; ++t) {
        const int64_t ext = a.r_mask[t] + 1, n = a.t_n[a.r_id[t]];
        filled *= (double)std::min(ext, n) / (double)ext;   // (a last partial tile along a long axis is ignored)
    }
}

template <class V>
void launch_tabcopy(const TabCopyArgs& ta, int ept, dim3 grid, size_t lds, hipStream_t st) {
    if (ept <= 8) TFH_LAUNCH_TIMED((tabcopy_kernel<V, 8>), grid, dim3(THREADS), lds, st, ta);
    else if (ept <= 16) TFH_LAUNCH_TIMED((tabcopy_kernel<V, 16>), grid, dim3(THREADS), lds, st, ta);
    else TFH_LAUNCH_TIMED((tabcopy_kernel<V, 32>), grid, dim3(THREADS), lds, st, ta);
}

// ---- long extents that are no powers of two ---------------------------------------------------------------------------
// A permutation of a tensor like [27,466,1401] has runs of kilobytes on both sides, but no power-of-two tile grid
// fits it, and a tile small enough to keep per-element offsets in registers has runs of a few hundred bytes that
// start anywhere: every run pays for the partly used 128-byte lines at its ends.  Here a tile is 64 KB and two-sided:
// a group RF of axes that are dense in the input (whole axes and, last, a range of the next one) and a group WF that
// is dense in the output.  A wave reads 64 consecutive elements of an input run per instruction -- thread t always
// has column 64 k + t of the run, the row changes with the register -- and writes them to LDS in read order; then it
// writes 64 consecutive elements of an output run per instruction, thread t gathering column 64 k + t of the
// write order from LDS.  What changes from row to row is the same for all lanes (the offset of the row in memory,
// the coordinates of the ranged axes it lies at) and comes from small tables that every block computes for itself
// in LDS at start: nothing is kept per element, so the tile can be large.  Tiles are full except at the last range
// of a ranged axis (two such axes at most), where lanes past the run's end and rows past the edge are left out of
// the stores; their loads are redirected to addresses inside the tile, so that no load is conditional.
constexpr int PERM_AXES = 8;   // axes per group
struct PermGroup {
    int32_t n;
    int32_t ext[PERM_AXES];    // mixed radix, innermost first
    int32_t lds[PERM_AXES];    // LDS position stride
    int32_t slot[PERM_AXES];   // 1, 2: the axis is ranged axis 1, 2
    int64_t mem[PERM_AXES];    // memory stride (elements)
};
struct PermArgs {
    const void* in;
    void* out;
    PermGroup rs, ws, wf;      // rows of the read order (input strides), rows of the write order (output strides), write columns
    int32_t rfn, rsn, wfn, wsn, pitch;
    int32_t nsegs, units;      // wave instructions per row of the read order, and in a tile
    int32_t conj;              // complex elements: the sign of the imaginary part is flipped on the way (the only change to the bits)
    int32_t rf_slot, wf_slot;  // the ranged axis that is last in RF / WF (0: none), and the elements per index of it
    int32_t rf_row, wf_row;
    int32_t x_n[2], x_t[2];    // extent of a ranged axis and its indices per tile (1, 1 when there is none)
    int32_t ng;
    int64_t ntiles;
    int64_t g_count[MAXG], g_si[MAXG], g_so[MAXG];
    int32_t g_slot[MAXG];
};

// entry i of a group: memory offset, LDS position, coordinates along the ranged axes (16 bits each)
__device__ __forceinline__ void perm_entry(const PermGroup& g, int i, uint32_t& mem, uint32_t& lds, uint32_t& xc) {
    int64_t m = 0;
    lds = xc = 0;
    for (int t = 0; t < g.n; ++t) {
        const int q = i / g.ext[t], c = i - q * g.ext[t];
        i = q;
        m += (int64_t)c * g.mem[t];
        lds += (uint32_t)(c * g.lds[t]);
        if (g.slot[t]) xc |= (uint32_t)c << (16 * (g.slot[t] - 1));
    }
    mem = (uint32_t)m;
}

constexpr int PERM_THREADS = 512, PERM_WAVES = PERM_THREADS / 64;
constexpr int PERM_WSEG = 8;   // a write run held in registers is up to 8 wave instructions wide

// The read order is dealt to the waves in units of one wave instruction: unit u is segment u % nsegs (64 columns) of
// row u / nsegs, wave w has units w, w + 8, ... in registers 0, 1, ...  What a unit needs (the offset of its row in
// memory, its first column, its place in LDS, the coordinates of its row along the ranged axes) is the same for all
// lanes: lane j of the wave computes it for the unit of register j once per block, and the loops below fetch it with
// a lane read.  A read run of any length is covered to within one instruction, whatever its extent.
// WTAB: the write run is longer than PERM_WSEG wave instructions (a short innermost axis of the output inside a longer
// dense run: batched transposes of small matrices): its LDS positions come from the table in LDS instead of registers,
// and the (row, segment) pairs of the write order are dealt to the waves one by one.
// W: elements per lane of a read instruction (2 for 8-byte elements when the read run is longer than one instruction
// of single elements: half the load and LDS-write instructions; the pair starts at any element, so its load is aligned
// to the element only and its two LDS writes are one ds_write2).
template <class V> struct PermPair;
template <> struct PermPair<uint32_t> { typedef uint32_t type __attribute__((ext_vector_type(2), aligned(4))); };
template <> struct PermPair<uint64_t> { typedef uint64_t type __attribute__((ext_vector_type(2), aligned(8))); };
template <> struct PermPair<double2> { typedef uint64_t type __attribute__((ext_vector_type(2), aligned(8))); };   // (never used: W = 1)

template <class V, int EPT, bool WTAB, int W = 1>
__global__ void __launch_bounds__(PERM_THREADS, WTAB ? 8 : (sizeof(V) == 4 ? 6 : 4)) perm_kernel(PermArgs a) {   // (waves per SIMD: four blocks per CU of the table's, else three of 4-byte elements, two of longer ones)
    prefetch_kernel_arguments<sizeof(PermArgs)>();
    extern __shared__ __align__(16) unsigned char smem_raw[];
    V* lds = reinterpret_cast<V*>(smem_raw);
    uint32_t* lw_f = reinterpret_cast<uint32_t*>(smem_raw + (size_t)a.pitch * a.rsn * sizeof(V));   // [wfn] LDS position of a column of the write order
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // the unit of register `lane` of this wave, the same in every tile
    uint32_t u_mem = 0, u_col = 0x40000000u, u_lds = 0, u_xc = 0xffffffffu;   // (no unit: past every run, never inside)
    {
        const int u = wave + PERM_WAVES * lane;
        if (lane < EPT / W && u < a.units) {
            const int r = u / a.nsegs, k = u - r * a.nsegs;
            uint32_t l;
            perm_entry(a.rs, r, u_mem, l, u_xc);
            u_col = (uint32_t)(64 * W * k);
            u_lds = l + u_col;
        }
    }
    const int my_units = __builtin_amdgcn_readfirstlane(a.units > wave ? (a.units - wave + PERM_WAVES - 1) / PERM_WAVES : 0);
    auto of_unit = [](uint32_t v, int j) { return (uint32_t)__builtin_amdgcn_readlane((int)v, j); };
    auto origin = [&](uint32_t tile, int64_t& oi, int64_t& oo, uint32_t& lim) {   // (tile counts are below 2^31)
        oi = oo = 0;
        int l[2] = {a.x_t[0], a.x_t[1]};
        for (int g = 0; g < a.ng; ++g) {
            const uint32_t n = (uint32_t)a.g_count[g], q = tile / n;
            const int64_t c = (int64_t)(tile - q * n);
            tile = q;
            oi += c * a.g_si[g];
            oo += c * a.g_so[g];
#pragma unroll
            for (int x = 0; x < 2; ++x)
                if (a.g_slot[g] == x + 1) {
                    const int64_t left = (int64_t)a.x_n[x] - c * a.x_t[x];
                    if (left < l[x]) l[x] = (int)left;
                }
        }
        oi = uniform64(oi);
        oo = uniform64(oo);
        lim = (uint32_t)__builtin_amdgcn_readfirstlane(l[0] | (l[1] << 16));
    };
    const uint32_t lim_full = (uint32_t)(a.x_t[0] | (a.x_t[1] << 16));
    auto inside = [&](uint32_t xc, uint32_t lim) { return (xc & 0xffffu) < (lim & 0xffffu) && (xc >> 16) < (lim >> 16); };
    auto run_len = [&](int slot, int row, int full, uint32_t lim) {   // elements of a run inside the tensor at this tile
        if (slot == 0) return full;
        return (int)(slot == 1 ? (lim & 0xffffu) : (lim >> 16)) * row;
    };
    // (a scalar base and a 32-bit byte offset per lane: the address of a load or store takes no registers of its own)
    auto at = [](auto* base, uint32_t i) {
        using T = std::remove_pointer_t<decltype(base)>;
        using B = std::conditional_t<std::is_const<T>::value, const char, char>;
        return reinterpret_cast<T*>(reinterpret_cast<B*>(base) + i * (uint32_t)sizeof(T));
    };
    // conjugation: the top bit of the last 32-bit word of a complex element (zero otherwise: a move of the bits)
    const uint32_t sign = (sizeof(V) >= 8 && a.conj) ? 0x80000000u : 0u;
    auto flip = [&](V v) {
        if constexpr (sizeof(V) >= 8) {
            uint32_t w[sizeof(V) / 4];
            __builtin_memcpy(w, &v, sizeof(V));
            w[sizeof(V) / 4 - 1] ^= sign;
            __builtin_memcpy(&v, w, sizeof(V));
        }
        return v;
    };
    V regs[EPT];
    // No load is conditional: a column past the end of the run reads the run's last element, a row past the edge of
    // the tensor reads row 0 of the tile, which lies inside at every tile.
    auto load = [&](int64_t oi, uint32_t lim, uint32_t z) {
        const V* in = reinterpret_cast<const V*>(a.in) + oi;
        const uint32_t last = (uint32_t)run_len(a.rf_slot, a.rf_row, a.rfn, lim) - 1u;
        // per unit, in the lane of its register: the row's offset at this tile, and the first column
        const uint32_t t_mem = inside(u_xc, lim) ? u_mem : 0u, t_col = u_col | z;
#pragma unroll
        for (int g = 0; g < EPT / W; g += 8) {
            if (g < my_units) {   // (eight units at a time: the last ones of a wave may be none, and read row 0)
#pragma unroll
                for (int j = g; j < g + 8; ++j) {
                    const V* row = in + of_unit(t_mem, j);
                    if constexpr (W == 1) {
                        const uint32_t col = min(of_unit(t_col, j) + (uint32_t)lane, last);
                        regs[j] = load_stream<Pack<V, 1>>(at(row, col)).v[0];
                    } else {
                        // a pair that starts at the run's last element is read one element earlier (its second
                        // element is the one wanted); runs are 16 elements and more
                        typedef typename PermPair<V>::type Pair;
                        const uint32_t col = of_unit(t_col, j) + 2u * (uint32_t)lane, from = min(col, last - 1u);
                        const Pair pr = __builtin_nontemporal_load(reinterpret_cast<const Pair*>(at(row, from)));
                        regs[2 * j] = col > from ? (V)pr[1] : (V)pr[0];
                        regs[2 * j + 1] = (V)pr[1];
                    }
                }
            }
        }
    };
    const uint32_t ntiles = (uint32_t)a.ntiles, per_xcd = (ntiles + 7) / 8, slots = per_xcd * 8;
    auto tile_of = [&](uint32_t slot) { return (slot & 7) * per_xcd + (slot >> 3); };   // every XCD a contiguous eighth
    uint32_t slot = blockIdx.x;
    while (slot < slots && tile_of(slot) >= ntiles) slot += gridDim.x;
    if (slot >= slots) return;
    int64_t oi, oo;
    uint32_t lim;
    origin(tile_of(slot), oi, oo, lim);
    load(oi, lim, tile_of(slot) >> 31);
    // (what the write phase needs is computed while the first tile's loads are in flight)
    for (int i = tid; i < a.wfn; i += PERM_THREADS) {
        uint32_t m, xc;
        perm_entry(a.wf, i, m, lw_f[i], xc);
    }
    // The write order the same way, one entry per lane: wave w has rows w, w + 8, ... of the write order (the offset
    // of the row in the output, its LDS position, its coordinates); WTAB: units of one wave instruction, segment
    // u % nsegw of row u / nsegw.  64 entries per wave at most.
    uint32_t w_out = 0, w_col = 0x40000000u, w_lrow = 0, w_xc = 0xffffffffu;
    int my_wunits;
    {
        const int nsegw = WTAB ? (a.wfn + 63) / 64 : 1, wunits = a.wsn * nsegw, u = wave + PERM_WAVES * lane;
        if (u < wunits) {
            const int ws = u / nsegw, k = u - ws * nsegw;
            perm_entry(a.ws, ws, w_out, w_lrow, w_xc);
            w_col = (uint32_t)(64 * k);
        }
        my_wunits = __builtin_amdgcn_readfirstlane(wunits > wave ? (wunits - wave + PERM_WAVES - 1) / PERM_WAVES : 0);
    }
    __syncthreads();
    uint32_t lwf[PERM_WSEG];   // LDS position of this thread's columns of the write order
#pragma unroll
    for (int k = 0; k < PERM_WSEG; ++k) lwf[k] = (!WTAB && 64 * k + lane < a.wfn) ? lw_f[64 * k + lane] : 0u;
    for (;;) {
        {
            const uint32_t z = tile_of(slot) >> 31, t_col = u_col | z, t_lds = u_lds | z;
#pragma unroll
            for (int g = 0; g < EPT / W; g += 8) {
                if (g < my_units) {
#pragma unroll
                    for (int j = g; j < g + 8; ++j) {
                        if constexpr (W == 1) {
                            if (of_unit(t_col, j) + (uint32_t)lane < (uint32_t)a.rfn) lds[of_unit(t_lds, j) + (uint32_t)lane] = flip(regs[j]);
                        } else {
                            const uint32_t col = of_unit(t_col, j) + 2u * (uint32_t)lane, pos = of_unit(t_lds, j) + 2u * (uint32_t)lane;
                            if (col + 1u < (uint32_t)a.rfn) {
                                lds[pos] = flip(regs[2 * j]);
                                lds[pos + 1u] = flip(regs[2 * j + 1]);
                            } else if (col < (uint32_t)a.rfn) {
                                lds[pos] = flip(regs[2 * j]);
                            }
                        }
                    }
                }
            }
        }
        __syncthreads();
        uint32_t next = slot + gridDim.x;
        while (next < slots && tile_of(next) >= ntiles) next += gridDim.x;
        const bool more = next < slots;
        int64_t oi2 = 0, oo2 = 0;
        uint32_t lim2 = 0;
        if (more) {   // the next tile's loads are in flight while this one is written out
            origin(tile_of(next), oi2, oo2, lim2);
            load(oi2, lim2, tile_of(next) >> 31);
        }
        V* out = reinterpret_cast<V*>(a.out) + oo;
        if (WTAB) {
            const uint32_t wlen = (uint32_t)run_len(a.wf_slot, a.wf_row, a.wfn, lim);
            const bool full = lim == lim_full;
            int j = 0;
            if (full) {   // (four units at a time: their LDS reads are in flight together)
                for (; j + 4 <= my_wunits; j += 4) {
                    uint32_t col[4], pos[4];
                    V v[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        col[i] = of_unit(w_col, j + i) + (uint32_t)lane;
                        pos[i] = col[i] < wlen ? lw_f[col[i]] : 0u;
                    }
#pragma unroll
                    for (int i = 0; i < 4; ++i) v[i] = lds[pos[i] + of_unit(w_lrow, j + i)];
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        if (col[i] < wlen) *at(out + of_unit(w_out, j + i), col[i]) = v[i];
                }
            }
            for (; j < my_wunits; ++j) {
                if (!full && !inside(of_unit(w_xc, j), lim)) continue;
                const uint32_t col = of_unit(w_col, j) + (uint32_t)lane;
                if (col < wlen) *at(out + of_unit(w_out, j), col) = lds[lw_f[col] + of_unit(w_lrow, j)];
            }
        } else if (lim == lim_full) {
            // a segment of the write run at a time: its guard is looked at once per tile, not once per row
#pragma unroll
            for (int k = 0; k < PERM_WSEG; ++k) {
                if (64 * k >= a.wfn) break;
                if (64 * k + lane < a.wfn) {
                    const uint32_t wcol = (uint32_t)(64 * k + lane);
                    // (a cached store: the next instruction completes the 128-byte lines this one leaves partly written)
                    // (a few rows at a time: their LDS reads are in flight together)
                    constexpr int WU = sizeof(V) == 4 ? 2 : 4;   // (what the registers leave)
                    int j = 0;
                    for (; j + WU <= my_wunits; j += WU) {
                        V v[WU];
#pragma unroll
                        for (int i = 0; i < WU; ++i) v[i] = lds[lwf[k] + of_unit(w_lrow, j + i)];
#pragma unroll
                        for (int i = 0; i < WU; ++i) *at(out + of_unit(w_out, j + i), wcol) = v[i];
                    }
                    for (; j < my_wunits; ++j) *at(out + of_unit(w_out, j), wcol) = lds[lwf[k] + of_unit(w_lrow, j)];
                }
            }
        } else {
            const int wlen = run_len(a.wf_slot, a.wf_row, a.wfn, lim);
#pragma unroll
            for (int k = 0; k < PERM_WSEG; ++k) {
                if (64 * k >= wlen) break;
                if (64 * k + lane < wlen) {
                    const uint32_t wcol = (uint32_t)(64 * k + lane);
                    for (int j = 0; j < my_wunits; ++j)
                        if (inside(of_unit(w_xc, j), lim)) *at(out + of_unit(w_out, j), wcol) = lds[lwf[k] + of_unit(w_lrow, j)];
                }
            }
        }
        if (!more) break;
        __syncthreads();
        slot = next;
        oo = oo2;
        lim = lim2;
    }
}

template <class V, int EPT>
void launch_perm(const PermArgs& pa, bool wtab, int w, dim3 grid, size_t lds, hipStream_t st) {
    if constexpr (sizeof(V) <= 8) {
        if (w == 2) {
            if (wtab) TFH_LAUNCH_TIMED((perm_kernel<V, EPT, true, 2>), grid, dim3(PERM_THREADS), lds, st, pa);
            else TFH_LAUNCH_TIMED((perm_kernel<V, EPT, false, 2>), grid, dim3(PERM_THREADS), lds, st, pa);
            return;
        }
    }
    if (wtab) TFH_LAUNCH_TIMED((perm_kernel<V, EPT, true>), grid, dim3(PERM_THREADS), lds, st, pa);
    else TFH_LAUNCH_TIMED((perm_kernel<V, EPT, false>), grid, dim3(PERM_THREADS), lds, st, pa);
}

// A bit-exact move of extents that the shift-and-mask tiles do not fill: two-sided 64 KB tiles.  Returns true when
// it launched (status holds the outcome).
struct PermPlan {
    PermArgs pa;
    bool wtab;
    int w;          // elements per lane of a read instruction
    size_t lds;
    dim3 grid;
    double score;   // bytes of the shorter of the two runs, each counted up to 1 KB, and how full the tile is
};
// One candidate tiling: a read run of up to rf_cap elements, a write run of up to wf_cap.
bool plan_perm_tiles(int eb, const void* in, void* out, std::vector<Axis> axes, int64_t rf_cap, int64_t wf_cap, double gain, PermPlan& plan) {
    int64_t total = 1;
    for (auto& x : axes) total *= x.n;
    if (total * eb < ((int64_t)8 << 20)) return false;   // (8 MB: below, the table tiles of 2048 elements measure the same or better)
    std::stable_sort(axes.begin(), axes.end(), [](const Axis& x, const Axis& y) { return std::llabs(x.s[1]) > std::llabs(y.s[1]); });
    fuse_axes(axes, 2);
    const int na = (int)axes.size();
    if (na < 2 || na > MAXG) return false;
    for (auto& x : axes)
        if (x.s[0] <= 0 || x.s[1] <= 0 || x.n > 0x7fffffff) return false;
    std::vector<int> in_order(na), out_order(na);
    for (int i = 0; i < na; ++i) in_order[i] = out_order[i] = i;
    std::stable_sort(in_order.begin(), in_order.end(), [&](int x, int y) { return axes[x].s[0] < axes[y].s[0]; });
    std::stable_sort(out_order.begin(), out_order.end(), [&](int x, int y) { return axes[x].s[1] < axes[y].s[1]; });
    if (axes[in_order[0]].s[0] != 1 || axes[out_order[0]].s[1] != 1) return false;
    const int ept = eb == 4 ? 32 : (eb == 8 ? 16 : 8);   // the registers of 512 threads hold a 64 KB tile
    // (a tensor too small to give every block that fits on the chip a tile of 64 KB takes smaller ones, down to
    // 16 KB: three quarters of the blocks, since the ragged ranges of the axes add tiles; half of them, or a balance
    // term in the score for a few tiles more than blocks, measured no better)
    const int64_t resident = 256 * (eb == 4 ? 3 : 2);
    const int64_t cap_bytes = std::min<int64_t>((int64_t)PERM_THREADS * ept * eb, std::max<int64_t>(16384, total * eb * 4 / (resident * 3)));
    int64_t emax = cap_bytes / eb;
    std::vector<int64_t> in_tile(na, 0);   // indices of the axis per tile (0: outside the tile)
    int nranged = 0;
    // the range of an axis of extent n behind `run` elements of whole axes, `room` indices at most: the one that
    // covers the axis in the fewest wave instructions (64 elements each, a last partial one per run), the longest of those
    auto best_range = [gain](int64_t n, int64_t run, int64_t room, bool other_run) {
        auto cost = [&](int64_t t) {   // wave instructions per element of the axis, both sides
            double per = (double)((run * t + 63) / 64) / (double)(run * t);
            if (other_run) per += (double)((t + 63) / 64) / (double)t;   // (the axis is the innermost of the other side)
            return per * (double)(t * ((n + t - 1) / t));
        };
        int64_t best_t = room;
        double best_cost = cost(room);
        for (int64_t t = room - 1; t >= std::max<int64_t>(2, room / 4); --t) {
            const double c = cost(t);
            if (c < best_cost * gain) {   // (a shorter range makes the tile smaller: `gain` is what it has to save)
                best_cost = c;
                best_t = t;
            }
        }
        const int64_t pieces = (n + best_t - 1) / best_t;   // (equal pieces, when that costs no more)
        const int64_t even = (n + pieces - 1) / pieces;
        if (cost(even) <= best_cost) best_t = even;
        return best_t;
    };
    // a dense run of up to `cap` elements along one side's order: whole axes, then a range of the next
    auto take_run = [&](int side, int64_t cap, int64_t& E, std::vector<char>& members) {
        const std::vector<int>& ord = side ? out_order : in_order;
        int64_t run = 1;
        for (int i : ord) {
            if (axes[i].s[side] != run) break;
            if (in_tile[i]) {   // already in the tile through the other side
                if (run * in_tile[i] > cap) break;
                members[i] = 1;
                run *= in_tile[i];
                if (in_tile[i] != axes[i].n) break;
                continue;
            }
            const int64_t room = std::min<int64_t>(cap / run, emax / E);
            if (axes[i].n <= room) {
                in_tile[i] = axes[i].n;
                members[i] = 1;
                E *= axes[i].n;
                run *= axes[i].n;
                continue;
            }
            if (room >= 2 && nranged < 2) {
                in_tile[i] = best_range(axes[i].n, run, room, axes[i].s[side ^ 1] == 1);
                members[i] = 1;
                E *= in_tile[i];
                run *= in_tile[i];
                ++nranged;
            }
            break;
        }
        return run;
    };
    int64_t E = 1;
    std::vector<char> in_rf(na, 0), in_wf(na, 0);
    // the read run first: two wave instructions wide at most (half that for 16-byte elements), then the write run in
    // the room that the registers of a thread leave (a row per wave and register)
    const int64_t rfn = take_run(0, rf_cap, E, in_rf);
    if (rfn < 16) return false;
    const int64_t nsegs = (rfn + 63) / 64, max_units = (int64_t)PERM_WAVES * ept;
    if (nsegs > max_units) return false;
    emax = std::min<int64_t>(emax, rfn * (max_units / nsegs));
    const int64_t wfn = take_run(1, wf_cap, E, in_wf);
    if (wfn < 16) return false;
    // room left (a short output run): more of the input's fastest axes, then whole axes from either side
    for (int side = 0, idle = 0; E * 2 <= emax && idle < 2; side ^= 1) {
        const std::vector<int>& ord = side ? out_order : in_order;
        int pick = -1;
        for (int i : ord)
            if (!in_tile[i]) { pick = i; break; }
        if (pick < 0) { ++idle; continue; }
        const int64_t room = emax / E;
        if (axes[pick].n <= room) {
            in_tile[pick] = axes[pick].n;
            E *= axes[pick].n;
            idle = 0;
        } else if (room >= 2 && nranged < 2) {
            const int64_t pieces = (axes[pick].n + room - 1) / room;
            in_tile[pick] = (axes[pick].n + pieces - 1) / pieces;
            E *= in_tile[pick];
            ++nranged;
            idle = 0;
        } else {
            ++idle;
        }
    }
    if (E * eb * 4 < cap_bytes) return false;   // (a quarter of the tile at least)
    PermArgs& pa = plan.pa;
    std::memset(&pa, 0, sizeof pa);
    pa.x_n[0] = pa.x_n[1] = pa.x_t[0] = pa.x_t[1] = 1;
    std::vector<int> slot(na, 0);
    int nslots = 0;
    for (int i = 0; i < na; ++i)
        if (in_tile[i] && in_tile[i] != axes[i].n) {
            slot[i] = ++nslots;
            pa.x_n[nslots - 1] = (int32_t)axes[i].n;
            pa.x_t[nslots - 1] = (int32_t)in_tile[i];
            if (in_tile[i] > 0xffff) return false;
        }
    // a ranged axis is the last of its run: the elements per index of it
    pa.rf_row = pa.wf_row = 1;
    for (int i : in_order)
        if (in_rf[i]) {
            if (slot[i]) pa.rf_slot = slot[i];
            else pa.rf_row *= (int32_t)in_tile[i];
        }
    for (int i : out_order)
        if (in_wf[i]) {
            if (slot[i]) pa.wf_slot = slot[i];
            else pa.wf_row *= (int32_t)in_tile[i];
        }
    const int64_t wfn2 = wfn;
    const int64_t rsn = E / rfn, wsn = E / wfn2;
    if (rsn * nsegs > max_units) return false;
    const int64_t pitch = rfn | 1;
    // LDS position strides: an axis of RF by its place in the run, a row axis by its place among the rows times the pitch
    std::vector<int64_t> lpos(na, 0);
    {
        int64_t f = 1, r = 1;
        for (int i : in_order) {
            if (!in_tile[i]) continue;
            if (in_rf[i]) {
                lpos[i] = f;
                f *= in_tile[i];
            }
        }
        for (int i : in_order) {
            if (!in_tile[i] || in_rf[i]) continue;
            lpos[i] = r * pitch;
            r *= in_tile[i];
        }
    }
    int64_t span_in = 0, span_out = 0;
    auto add = [&](PermGroup& g, int i, int64_t mem) {
        if (g.n == PERM_AXES) return false;
        g.ext[g.n] = (int32_t)in_tile[i];
        g.lds[g.n] = (int32_t)lpos[i];
        g.slot[g.n] = slot[i];
        g.mem[g.n] = mem;
        ++g.n;
        return true;
    };
    for (int i : in_order) {
        if (!in_tile[i]) continue;
        span_in += (in_tile[i] - 1) * axes[i].s[0];
        span_out += (in_tile[i] - 1) * axes[i].s[1];
        if (!in_rf[i] && !add(pa.rs, i, axes[i].s[0])) return false;
    }
    for (int i : out_order) {
        if (!in_tile[i]) continue;
        if (in_wf[i]) {
            if (!add(pa.wf, i, axes[i].s[1])) return false;
        } else if (!add(pa.ws, i, axes[i].s[1])) {
            return false;
        }
    }
    if (span_in >= ((int64_t)1 << 32) || span_out >= ((int64_t)1 << 32)) return false;   // 32-bit element offsets
    pa.rfn = (int32_t)rfn;
    pa.rsn = (int32_t)rsn;
    pa.wfn = (int32_t)wfn2;
    pa.wsn = (int32_t)wsn;
    pa.pitch = (int32_t)pitch;
    pa.nsegs = (int32_t)nsegs;
    pa.units = (int32_t)(rsn * nsegs);
    // pairs per lane in the read phase: a read run of more than one instruction of single elements, rows that still
    // fit the registers, and no tile whose read run is a single element (the pair would reach past it)
    plan.w = 1;
    {
        const int64_t nsegs2 = (rfn + 127) / 128;
        bool short_run = false;
        if (pa.rf_slot) {
            const int64_t n = pa.x_n[pa.rf_slot - 1], t = pa.x_t[pa.rf_slot - 1];
            short_run = (n % t) * pa.rf_row == 1;
        }
        if (eb == 8 && rfn > 64 && rsn * nsegs2 <= max_units / 2 && !short_run) {   // (4-byte elements measured 2 points slower with pairs, 8-byte ones 3 faster)
            plan.w = 2;
            pa.nsegs = (int32_t)nsegs2;
            pa.units = (int32_t)(rsn * nsegs2);
        }
    }
    pa.in = in;
    pa.out = out;
    int64_t ntiles = 1;
    // the order of the tiles: fastest the innermost axis of the output that leaves the tile (the tiles that complete
    // the 128-byte lines at the ends of the write runs follow at once), then the innermost such axis of the input (the
    // same for the read runs, a few tiles later: tiles in flight on an XCD at the same time share its L2), then the
    // rest from the output's fast end
    std::vector<int> g_order;
    for (int i = na - 1; i >= 0; --i)
        if (in_tile[i] != axes[i].n) g_order.push_back(i);
    if (g_order.size() > 2) {
        size_t pick = 1;
        for (size_t k = 2; k < g_order.size(); ++k)
            if (axes[g_order[k]].s[0] < axes[g_order[pick]].s[0]) pick = k;
        const int moved = g_order[pick];
        g_order.erase(g_order.begin() + (long)pick);
        g_order.insert(g_order.begin() + 1, moved);
    }
    for (int i : g_order) {
        const int64_t t = in_tile[i] ? in_tile[i] : 1, count = (axes[i].n + t - 1) / t;
        if (pa.ng == MAXG) return false;
        pa.g_count[pa.ng] = count;
        pa.g_si[pa.ng] = axes[i].s[0] * t;
        pa.g_so[pa.ng] = axes[i].s[1] * t;
        pa.g_slot[pa.ng] = slot[i];
        ++pa.ng;
        ntiles *= count;
    }
    pa.ntiles = ntiles;
    if (ntiles < 256 || ntiles >= ((int64_t)1 << 31) - 8) return false;   // (a tile per CU at least)
    const bool wtab = wfn2 > 64 * PERM_WSEG;
    if (wsn * (wtab ? (wfn2 + 63) / 64 : 1) > PERM_THREADS) return false;   // (a lane of a wave per row or unit of the write order)
    const size_t lds = (size_t)pitch * rsn * eb + (size_t)wfn2 * sizeof(uint32_t);
    if (lds > 150 * 1024) return false;
    // (blocks per CU: by LDS, and by the registers that the kernels are compiled for)
    const size_t per_cu = std::max<size_t>(1, std::min<size_t>(wtab ? 4 : (eb == 4 ? 3 : 2), (size_t)(160 * 1024) / (lds + 512)));
    plan.wtab = wtab;
    plan.lds = lds;
    plan.grid = dim3((uint32_t)std::min<int64_t>((ntiles + 7) / 8 * 8, (int64_t)(256 * per_cu)));   // (a multiple of 8: a block stays on its XCD)
    // the share of the lanes of the wave instructions that move an element: last partial instructions of a run, last
    // partial ranges of an axis
    double lanes = ((double)rfn / (double)(64 * nsegs)) * ((double)wfn2 / (double)(64 * ((wfn2 + 63) / 64)));
    for (int i = 0; i < na; ++i)
        if (in_tile[i] && in_tile[i] != axes[i].n) lanes *= (double)axes[i].n / (double)(in_tile[i] * ((axes[i].n + in_tile[i] - 1) / in_tile[i]));
    // the lanes of a write instruction gather along the innermost axis of the write run: an even LDS stride there
    // has them collide in the banks
    const int64_t gather = pa.wf.n ? pa.wf.lds[0] : 1;
    const double banks = (gather & 1) ? 1.0 : ((gather & 3) ? 0.8 : 0.6);
    // What the measurements of odd shapes show, as factors: a read run pays for the partly used 128-byte lines at its
    // ends (the tiles that follow complete those of a write run); a tile in the table-driven write order reads LDS
    // once more per element; 4-byte elements are bound by instruction issue and gain from a third block per CU, longer
    // ones from larger tiles; a single block per CU has nothing to overlap its two phases with; and the tiles of a CU
    // together should hold the ~96 KB that cover the memory latency.
    const double r_bytes = (double)(rfn * eb), w_bytes = (double)(wfn2 * eb);
    const double blocks = (double)per_cu;
    const double occupancy = per_cu == 1 ? 0.72 : (eb == 4 ? (per_cu == 2 ? 0.92 : 1.0) : (per_cu == 2 ? 1.0 : 0.97));
    const double in_flight = std::min(1.0, blocks * (double)(E * eb) / 98304.0);
    plan.score = 1000.0 * (r_bytes / (r_bytes + 128.0)) * (w_bytes / (w_bytes + 32.0)) * (wtab ? 0.85 : 1.0) * lanes * banks * occupancy *
                 (0.4 + 0.6 * in_flight);
    return true;
}

// A bit-exact move of extents that the shift-and-mask tiles do not fill: two-sided 64 KB tiles.  Returns true when
// it launched (status holds the outcome).
bool try_perm_tiles(int eb, const void* in, void* out, std::vector<Axis> axes, bool conj, void* stream, int32_t& status) {
    status = TFH_OK;
    // candidates: the usual read run (two wave instructions wide, one for 16-byte elements) or one twice as long (an
    // innermost axis that both sides share, with one long axis behind it: the read run is all that can grow), a write
    // run held in registers or a longer one through the table (a short innermost output axis inside a longer dense run)
    PermPlan best;
    best.score = 0.0;
    const int64_t rf0 = eb == 16 ? 64 : 128;
    // (the winner of an earlier call with the same extents and strides is kept: the candidates cost tens of us)
    struct Kept {
        std::vector<int64_t> key;
        PermPlan plan;
    };
    static std::mutex kept_mutex;
    static std::vector<Kept> kept;
    std::vector<int64_t> key;
    key.push_back(eb);
    for (auto& x : axes) {
        key.push_back(x.n);
        key.push_back(x.s[0]);
        key.push_back(x.s[1]);
    }
    bool found = false;
    {
        std::lock_guard<std::mutex> lock(kept_mutex);
        for (auto& k : kept)
            if (k.key == key) {
                best = k.plan;
                found = true;
                break;
            }
    }
    if (!found) {
        for (int64_t rf_cap : {rf0, 4 * rf0, 16 * rf0, (int64_t)16384})
            for (int64_t wf_cap : {(int64_t)64 * PERM_WSEG, (int64_t)8192})
                for (double gain : {0.999, 0.9}) {
                    PermPlan cand;
                    std::memset(&cand.pa, 0, sizeof cand.pa);
                    if (plan_perm_tiles(eb, in, out, axes, rf_cap, wf_cap, gain, cand) && cand.score > best.score * 1.02) best = cand;
                }
        std::lock_guard<std::mutex> lock(kept_mutex);
        if (kept.size() >= 64) kept.erase(kept.begin());
        kept.push_back(Kept{key, best});
    }
    best.pa.in = in;
    best.pa.out = out;
    best.pa.conj = conj ? 1 : 0;
    if (best.score <= 0.0) return false;
    static const bool lds_limit_raised = [] {
        const int cap = 160 * 1024;
#define TFH_PERM_LDS(V, E, W) \
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&perm_kernel<V, E, W>), hipFuncAttributeMaxDynamicSharedMemorySize, cap); \
    if constexpr (sizeof(V) <= 8) \
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&perm_kernel<V, E, W, 2>), hipFuncAttributeMaxDynamicSharedMemorySize, cap);
        TFH_PERM_LDS(uint32_t, 32, false)
        TFH_PERM_LDS(uint64_t, 16, false)
        TFH_PERM_LDS(double2, 8, false)
        TFH_PERM_LDS(uint32_t, 32, true)
        TFH_PERM_LDS(uint64_t, 16, true)
        TFH_PERM_LDS(double2, 8, true)
#undef TFH_PERM_LDS
        return true;
    }();
    (void)lds_limit_raised;
    hipStream_t st = (hipStream_t)stream;
    const int prof = prof_begin(PROF_COPY, stream);
    if (eb == 4) launch_perm<uint32_t, 32>(best.pa, best.wtab, best.w, best.grid, best.lds, st);
    else if (eb == 8) launch_perm<uint64_t, 16>(best.pa, best.wtab, best.w, best.grid, best.lds, st);
    else launch_perm<double2, 8>(best.pa, best.wtab, best.w, best.grid, best.lds, st);
    prof_end(prof, stream);
    status = hip_check(hipGetLastError(), "copy kernel launch");
    return true;
}

// A bit-exact move whose shift-and-mask tiles come out with short runs or mostly empty: tiles of whole axes, driven by
// tables.  Returns true when it launched (status holds the outcome).
bool try_table_copy(int eb, const void* in, void* out, std::vector<Axis> axes, const TilePlan& tp, void* stream, int32_t& status) {
    status = TFH_OK;
    int64_t total = 1;
    for (auto& x : axes) total *= x.n;
    if (total < 65536) return false;
    int64_t run_in_old, run_out_old;
    double filled;
    masked_plan_quality(tp.args, run_in_old, run_out_old, filled);
    const double old_q = (double)std::min<int64_t>(std::min(run_in_old, run_out_old) * eb, 512) * (tp.all_full ? 1.0 : filled);
    if (tp.all_full && old_q >= 256.0) return false;   // (tiles with a ragged edge pay a bounds check per element there)
    std::stable_sort(axes.begin(), axes.end(), [](const Axis& x, const Axis& y) { return std::llabs(x.s[1]) > std::llabs(y.s[1]); });
    fuse_axes(axes, 2);
    const int na = (int)axes.size();
    if (na < 2 || na > MAXG) return false;
    for (auto& x : axes)
        if (x.s[0] <= 0 || x.s[1] <= 0) return false;   // broadcast or reversed axes stay with the general path
    std::vector<int> in_order(na), out_order(na);
    for (int i = 0; i < na; ++i) in_order[i] = out_order[i] = i;
    std::stable_sort(in_order.begin(), in_order.end(), [&](int x, int y) { return axes[x].s[0] < axes[y].s[0]; });
    std::stable_sort(out_order.begin(), out_order.end(), [&](int x, int y) { return axes[x].s[1] < axes[y].s[1]; });
    // axes alternately from the input's and the output's fastest end while a side is short of `want`: whole while the
    // tile has room for them and for what the other side still needs, else a range of the axis, which closes the side
    // (eight elements per thread: with 16 or 32 the three offsets per element fill the register file and one block
    // is left per CU -- [5]^9 f64 reversed 46 us with 32, 36 with 16, 24 with 8)
    const int64_t emax = std::min<int64_t>(61440 / eb, (int64_t)THREADS * 8);
    const int64_t want = std::max<int64_t>(1, 512 / eb);
    std::vector<int64_t> in_tile(na, 0);   // indices of the axis per tile (0: outside the tile)
    int64_t E = 1, run[2] = {1, 1};
    size_t pos[2] = {0, 0};
    bool open_[2] = {true, true};
    int nranged = 0;
    const std::vector<int>* order[2] = {&in_order, &out_order};
    auto advance = [&](int side) {   // run of a side = product of the leading axes of its order that are in the tile
        while (open_[side] && pos[side] < (size_t)na && in_tile[(*order[side])[pos[side]]]) {
            const int i = (*order[side])[pos[side]];
            if (axes[i].s[side] != run[side]) { open_[side] = false; break; }   // not contiguous with the run so far
            run[side] *= in_tile[i];
            if (in_tile[i] != axes[i].n) { open_[side] = false; break; }         // a range ends the run
            ++pos[side];
        }
        if (pos[side] == (size_t)na) open_[side] = false;
    };
    for (;;) {
        advance(0);
        advance(1);
        int side = -1;
        if (open_[0] && run[0] < want && (!(open_[1] && run[1] < want) || run[0] <= run[1])) side = 0;
        else if (open_[1] && run[1] < want) side = 1;
        if (side < 0) break;
        const int i = (*order[side])[pos[side]];
        if (axes[i].s[side] != run[side]) { open_[side] = false; continue; }
        const int other = side ^ 1;
        const int64_t need_other = (open_[other] && run[other] < want) ? (want + run[other] - 1) / run[other] : 1;
        const int64_t room = emax / E, fair = std::max<int64_t>(1, room / need_other);
        if (axes[i].n <= fair) {
            in_tile[i] = axes[i].n;
            E *= axes[i].n;
            continue;
        }
        // a range of it: the room that is left, less what the other side still needs
        const int64_t t0 = std::min<int64_t>(fair, 0xffff);
        // (extents that the shift-and-mask tiles fill completely keep those tiles' 16-byte accesses: whole axes only)
        if (t0 < 2 || nranged == 2 || tp.all_full) { open_[side] = false; continue; }
        const int64_t pieces = (axes[i].n + t0 - 1) / t0;
        in_tile[i] = (axes[i].n + pieces - 1) / pieces;
        E *= in_tile[i];
        ++nranged;
    }
    // runs reached with a small tile (a few short axes serve both sides): more whole axes, the input's innermost free
    // axis and the output's in turn, until a block has 2048 elements to move per tile
    for (int side = 0, idle = 0; E < 2048 && idle < 2; side ^= 1) {
        int pick = -1;
        for (int i : *order[side])
            if (!in_tile[i]) { pick = i; break; }
        if (pick < 0 || E * axes[pick].n > emax) { ++idle; continue; }
        idle = 0;
        in_tile[pick] = axes[pick].n;
        E *= axes[pick].n;
    }
    // the runs of the finished tile
    for (int side = 0; side < 2; ++side) {
        run[side] = 1;
        for (int i : *order[side]) {
            if (!in_tile[i] || axes[i].s[side] != run[side]) break;
            run[side] *= in_tile[i];
            if (in_tile[i] != axes[i].n) break;
        }
    }
    if (E < 512) return false;
    const double new_q = (double)std::min<int64_t>(std::min(run[0], run[1]) * eb, 512);
    if (tp.all_full && new_q < 2.0 * old_q) return false;   // (ragged shift-and-mask tiles lose more to their bounds checks than shorter runs cost)
    // tile axes in read order (with their LDS strides) and in write order
    TabBuildArgs tb;
    std::memset(&tb, 0, sizeof tb);
    TabCopyArgs ta;
    std::memset(&ta, 0, sizeof ta);
    ta.x_n[0] = ta.x_n[1] = ta.x_t[0] = ta.x_t[1] = 1;
    std::vector<int> rpos(na, 0), slot(na, 0);
    int nslots = 0;
    for (int i = 0; i < na; ++i)
        if (in_tile[i] && in_tile[i] != axes[i].n) {
            slot[i] = ++nslots;
            ta.x_n[nslots - 1] = (int32_t)axes[i].n;
            ta.x_t[nslots - 1] = (int32_t)in_tile[i];
            if (axes[i].n > 0x7fffffff) return false;
        }
    int64_t lo = 1, span_in = 0, span_out = 0;
    std::string key = "copytab|" + std::to_string(eb);
    for (int i : in_order)
        if (in_tile[i]) {
            if (tb.nt == TAB_MAX_AXES) return false;
            tb.r_ext[tb.nt] = (int32_t)in_tile[i];
            tb.r_si[tb.nt] = axes[i].s[0];
            tb.r_slot[tb.nt] = slot[i];
            rpos[i] = (int)lo;
            lo *= in_tile[i];
            ++tb.nt;
            span_in += (in_tile[i] - 1) * axes[i].s[0];
            span_out += (in_tile[i] - 1) * axes[i].s[1];
            key += "|" + std::to_string(in_tile[i]) + "," + std::to_string(axes[i].s[0]) + "," + std::to_string(axes[i].s[1]) + "," + std::to_string(slot[i]);
        }
    if (span_in >= ((int64_t)1 << 32) || span_out >= ((int64_t)1 << 32)) return false;   // 32-bit element offsets
    int w = 0;
    for (int i : out_order)
        if (in_tile[i]) {
            tb.w_ext[w] = (int32_t)in_tile[i];
            tb.w_so[w] = axes[i].s[1];
            tb.w_rpos[w] = rpos[i];
            tb.w_slot[w] = slot[i];
            ++w;
        }
    tb.E = (int32_t)E;
    ta.in = in;
    ta.out = out;
    ta.E = (int32_t)E;
    int64_t ntiles = 1;
    // the order of the tiles: fastest the innermost axis of the output that leaves the tile (the tiles that complete
    // the 128-byte lines at the ends of the write runs follow at once), then the innermost such axis of the input (the
    // same for the read runs, a few tiles later: tiles in flight on an XCD at the same time share its L2), then the
    // rest from the output's fast end
    std::vector<int> g_order;
    for (int i = na - 1; i >= 0; --i)
        if (in_tile[i] != axes[i].n) g_order.push_back(i);
    if (g_order.size() > 2) {
        size_t pick = 1;
        for (size_t k = 2; k < g_order.size(); ++k)
            if (axes[g_order[k]].s[0] < axes[g_order[pick]].s[0]) pick = k;
        const int moved = g_order[pick];
        g_order.erase(g_order.begin() + (long)pick);
        g_order.insert(g_order.begin() + 1, moved);
    }
    for (int i : g_order) {
        const int64_t t = in_tile[i] ? in_tile[i] : 1, count = (axes[i].n + t - 1) / t;
        if (ta.ng == MAXG) return false;
        ta.g_count[ta.ng] = count;
        ta.g_si[ta.ng] = axes[i].s[0] * t;
        ta.g_so[ta.ng] = axes[i].s[1] * t;
        ta.g_slot[ta.ng] = slot[i];
        ++ta.ng;
        ntiles *= count;
    }
    ta.ntiles = ntiles;
    if (ntiles < 8) return false;
    void* tab = nullptr;
    bool fresh = false;
    if ((status = table_cache_get(stream, key, (size_t)5 * E * sizeof(uint32_t), &tab, &fresh)) != TFH_OK) return true;
    if (!tab) return false;   // no cached block to be had (cache full, stream being captured): the masked tiles do it
    hipStream_t st = (hipStream_t)stream;
    if (fresh) {
        tb.tab = (uint32_t*)tab;
        hipLaunchKernelGGL(tabcopy_build_kernel, dim3((uint32_t)((E + THREADS - 1) / THREADS)), dim3(THREADS), 0, st, tb);
        table_cache_commit(stream, key);
    }
    ta.tab = (const uint32_t*)tab;
    const int ept = (int)((E + THREADS - 1) / THREADS);
    const size_t lds = (size_t)(E + E / 32 + 4) * eb;
    const size_t per_cu = std::max<size_t>(1, std::min<size_t>(4, (size_t)(160 * 1024) / (lds + 512)));
    const dim3 grid((uint32_t)std::min<int64_t>((ntiles + 7) / 8 * 8, (int64_t)(256 * per_cu)));   // (a multiple of 8: a block stays on its XCD)
    const int prof = prof_begin(PROF_COPY, stream);
    if (eb == 4) launch_tabcopy<uint32_t>(ta, ept, grid, lds, st);
    else if (eb == 8) launch_tabcopy<uint64_t>(ta, ept, grid, lds, st);
    else launch_tabcopy<double2>(ta, ept, grid, lds, st);
    prof_end(prof, stream);
    status = hip_check(hipGetLastError(), "copy kernel launch");
    return true;
}
}  // namespace

int32_t launch_copy(int dtype, const void* in, void* out, std::vector<Axis> axes, Scalar alpha, Scalar beta, bool conj,
                    void* stream) {
    const int eb = (int)dtype_size(dtype);
    if (!aligned(in, eb) || !aligned(out, eb)) return set_error(TFH_ERR_STRIDED, "view base is not aligned to the element size (%d bytes)", eb);
    for (auto& x : axes) x.s[2] = 0;
    TilePlan tp;
    const int max_tile = eb >= 16 ? 2048 : 4096;   // 32 KB of LDS per tile
    if (int32_t e = plan_tiles(axes, eb, max_tile, true, tp)) return e;
    if (tp.grid.x == 0) return TFH_OK;
    tp.args.in = in;
    tp.args.out = out;
    set_scalars(tp.args, alpha, beta, conj);
    hipStream_t st = (hipStream_t)stream;
    const bool vin = tp.vec_in && aligned(in, 16), vout = tp.vec_out && aligned(out, 16);
    const bool cx = is_complex(dtype);
    const bool raw = alpha.is_one() && beta.is_zero() && !(conj && cx);
    if (!raw && alpha.is_one() && beta.is_zero() && !tp.all_full) {   // a conjugating move: the two-sided tiles flip the sign on the way
        int32_t st_tab = TFH_OK;
        if (try_perm_tiles(eb, in, out, axes, true, stream, st_tab)) return st_tab;
    }
    if (raw) {
        int32_t st_tab = TFH_OK;
        if (!tp.all_full && try_perm_tiles(eb, in, out, axes, false, stream, st_tab)) return st_tab;
        if (try_table_copy(eb, in, out, axes, tp, stream, st_tab)) return st_tab;
        // Large tiles.  When the rows a tile touches on one side lie far apart (an axis that is contiguous on one side
        // and the slowest on the other: strides of megabytes inside every tile), 512-byte runs on that side cost 10-17 %
        // of the rate; four times the tile, spent on that side's run alone (2 KB), gets most of it back.
        if (tp.all_full && ((vin && vout) || eb == 16) && tp.args.tile_elems == max_tile) {
            int64_t far_[2] = {0, 0};
            for (int t = 0; t < tp.args.nt; ++t) {
                far_[0] = std::max<int64_t>(far_[0], std::llabs(tp.args.r_si[t]) * eb);
                far_[1] = std::max<int64_t>(far_[1], std::llabs(tp.args.w_so[t]) * eb);
            }
            const int side = far_[1] >= far_[0] ? 1 : 0;
            const bool want = far_[side] >= ((int64_t)1 << 20);
            TilePlan big;
            if (want && plan_tiles(axes, eb, max_tile, true, big, side, 2) == TFH_OK && big.all_full && ((big.vec_in && big.vec_out) || eb == 16) &&
                big.args.tile_elems == 4 * max_tile && big.args.ntiles >= 256 && big.args.ntiles < ((int64_t)1 << 30) && big.args.ng <= WALKG) {
                big.args.in = in;
                big.args.out = out;
                set_scalars(big.args, alpha, beta, conj);
                big.persistent = (uint32_t)std::min<int64_t>(big.args.ntiles, 256);
                const size_t lds = (size_t)(big.args.tile_elems + big.args.tile_elems / 32 + 4) * eb;
                const int prof = prof_begin(PROF_COPY, st);
                switch (eb) {
                    case 4: launch_copy_large<uint32_t, 32>(big, lds, st); break;
                    case 8: launch_copy_large<uint64_t, 32>(big, lds, st); break;
                    default: launch_copy_large<double2, 16>(big, lds, st); break;
                }
                prof_end(prof, st);
                return hip_check(hipGetLastError(), "copy kernel launch");
            }
            clear_error();
        }
        switch (eb) {
            case 4: return run_copy<uint32_t, RawOp<uint32_t>, true>(tp, RawOp<uint32_t>(), false, vin, vout, st);
            case 8: return run_copy<uint64_t, RawOp<uint64_t>, true>(tp, RawOp<uint64_t>(), false, vin, vout, st);
            default: return run_copy<double2, RawOp<double2>, false>(tp, RawOp<double2>(), false, vin, vout, st);
        }
    }
    const bool rb = !beta.is_zero();
    if (alpha.is_one() && beta.is_zero() && conj) {
        if (dtype == TFH_C64) return run_copy<float2, ConjOp<float2>, false>(tp, ConjOp<float2>(), false, vin, vout, st);
        return run_copy<double2, ConjOp<double2>, false>(tp, ConjOp<double2>(), false, vin, vout, st);
    }
    switch (dtype) {
        case TFH_F32: return run_copy<float, RealOp<float>, false>(tp, RealOp<float>(), rb, vin, vout, st);
        case TFH_F64: return run_copy<double, RealOp<double>, false>(tp, RealOp<double>(), rb, vin, vout, st);
        case TFH_C64: return run_copy<float2, CplxOp<float2, float>, false>(tp, CplxOp<float2, float>(), rb, vin, vout, st);
        default: return run_copy<double2, CplxOp<double2, double>, false>(tp, CplxOp<double2, double>(), rb, vin, vout, st);
    }
}

int32_t launch_fill(int dtype, void* out, std::vector<Axis> axes, Scalar value, void* stream) {
    const int eb = (int)dtype_size(dtype);
    if (!aligned(out, eb)) return set_error(TFH_ERR_STRIDED, "view base is not aligned to the element size (%d bytes)", eb);
    for (auto& x : axes) {  // slot 1 is the output everywhere in the tile planner
        x.s[1] = x.s[0];
        x.s[0] = x.s[2] = 0;
    }
    TilePlan tp;
    if (int32_t e = plan_tiles(axes, eb, 4096, false, tp)) return e;
    if (tp.grid.x == 0) return TFH_OK;
    tp.args.out = out;
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case TFH_F32: hipLaunchKernelGGL(fill_kernel<float>, tp.grid, dim3(THREADS), 0, st, tp.args, (float)value.re, tp.ept); break;
        case TFH_F64: hipLaunchKernelGGL(fill_kernel<double>, tp.grid, dim3(THREADS), 0, st, tp.args, value.re, tp.ept); break;
        case TFH_C64: hipLaunchKernelGGL(fill_kernel<float2>, tp.grid, dim3(THREADS), 0, st, tp.args, make_float2((float)value.re, (float)value.im), tp.ept); break;
        default: hipLaunchKernelGGL(fill_kernel<double2>, tp.grid, dim3(THREADS), 0, st, tp.args, make_double2(value.re, value.im), tp.ept); break;
    }
    return hip_check(hipGetLastError(), "fill kernel launch");
}

int32_t launch_emul(int dtype, const void* a, const void* b, void* c, std::vector<Axis> axes, Scalar alpha, Scalar beta,
                    void* stream) {
    // incoming slots: s[0]=A, s[1]=B, s[2]=C -> planner slots: 0 = A, 1 = output, 2 = B
    for (auto& x : axes) std::swap(x.s[1], x.s[2]);
    const int eb = (int)dtype_size(dtype);
    const int rb = is_double(dtype) ? 8 : 4;
    if (!aligned(a, rb) || !aligned(b, rb) || !aligned(c, rb)) return set_error(TFH_ERR_STRIDED, "view base is not aligned");
    // The tiles follow the contiguous axes of A and of the output.  A second operand whose contiguous axis is neither
    // of them would be read one element per sector (16^6 f64 with reversed modes: 168 us against 78 us): it is first
    // brought into the output's axis order by the tiled copy (one more pass over it at the copy kernel's rate).
    void* packed = nullptr;
    {
        int fast[3] = {-1, -1, -1};
        int64_t total = 1;
        for (size_t d = 0; d < axes.size(); ++d) {
            total *= axes[d].n;
            for (int slot = 0; slot < 3; ++slot)
                if (axes[d].n > 1 && std::llabs(axes[d].s[slot]) == 1) fast[slot] = (int)d;
        }
        bool scattered = total >= 65536 && fast[2] != fast[0] && fast[2] != fast[1];
        for (auto& x : axes)
            if (x.n > 1 && x.s[2] == 0) scattered = false;   // a broadcast operand is small: leave it alone
        if (scattered) {
            std::vector<size_t> order(axes.size());
            for (size_t d = 0; d < axes.size(); ++d) order[d] = d;
            std::stable_sort(order.begin(), order.end(), [&](size_t x, size_t y) { return std::llabs(axes[x].s[1]) > std::llabs(axes[y].s[1]); });
            std::vector<Axis> cp(axes.size());
            int64_t run = 1;
            for (size_t q = order.size(); q-- > 0;) {   // dense strides, the output's slowest axis outermost
                const size_t d = order[q];
                cp[d] = Axis{axes[d].n, {axes[d].s[2], run, 0}, axes[d].label};
                run *= axes[d].n;
            }
            if (int32_t e = pool_alloc(stream, (size_t)total * eb, &packed)) return e;
            Scalar one, zero;
            one.re = 1;
            if (int32_t e = launch_copy(dtype, b, packed, cp, one, zero, false, stream)) {
                pool_free(stream, packed);
                return e;
            }
            for (size_t d = 0; d < axes.size(); ++d) axes[d].s[2] = cp[d].s[1];
            b = packed;
        }
    }
    TilePlan tp;
    if (int32_t e = plan_tiles(axes, eb, 2048, false, tp)) {
        pool_free(stream, packed);
        return e;
    }
    if (tp.grid.x == 0) {
        pool_free(stream, packed);
        return TFH_OK;
    }
    tp.args.in = a;
    tp.args.in2 = b;
    tp.args.out = c;
    set_scalars(tp.args, alpha, beta, false);
    hipStream_t st = (hipStream_t)stream;
    switch (dtype) {
        case TFH_F32: TFH_LAUNCH_TIMED((emul_kernel<float, false>), tp.grid, dim3(THREADS), 0, st, tp.args, tp.ept); break;
        case TFH_F64: TFH_LAUNCH_TIMED((emul_kernel<double, false>), tp.grid, dim3(THREADS), 0, st, tp.args, tp.ept); break;
        case TFH_C64: TFH_LAUNCH_TIMED((emul_kernel<float, true>), tp.grid, dim3(THREADS), 0, st, tp.args, tp.ept); break;
        default: TFH_LAUNCH_TIMED((emul_kernel<double, true>), tp.grid, dim3(THREADS), 0, st, tp.args, tp.ept); break;
    }
    pool_free(stream, packed);   // stream-ordered: the block is reused only by later work on this stream
    return hip_check(hipGetLastError(), "elementwise kernel launch");
}

}  // namespace tfh
