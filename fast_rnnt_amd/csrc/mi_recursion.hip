// Lattice ("mutual information") recursion, forward and backward, for gfx950.
//
// Mapping.  One workgroup per utterance, one lane per lattice row.  A *sweep
// wave* owns 64 consecutive rows and walks the lattice along anti-diagonals: at
// local step e lane L works on column e - L, so the neighbour in the previous
// row is what lane L-1 produced one step earlier (regular lattice) or two steps
// earlier (modified lattice) and arrives through a DPP wave shift, and the
// neighbour in the same row is the lane's own previous result.
//
// A single wave issues about one instruction every 4.5 cycles (a dependent one every 8, a
// scalar test with its branch costs 18 cycles, 35 when taken) and nothing overlaps
// within it, so a sweep wave's time is its instruction count: everything that is not
// the dependent chain is kept off it, and tiles that need no tests run without them,
// each kind of tile in a loop of its own.  *Staging waves* of the same workgroup fetch
// px/py (forward) or p/px (backward) with coalesced, range-checked row loads, turn
// them into diagonal ("sheared") 64-row x 32-step tiles in LDS and -- for the
// backward sweep -- also evaluate the exp() of the gradient split; the sweep wave
// pulls a tile into registers with 16-byte LDS reads and leaves the tile's results
// in the same LDS buffer with 16-byte writes.  The staging waves carry the results
// to memory as coalesced row segments through range-checked buffer stores (a cell
// outside the window gets an offset that the hardware drops instead of a branch)
// once they have refilled the buffer.  There are two or three buffers per sweep wave;
// sweep and staging waves meet only through monotone LDS counters (bounded
// spinning; one counter per buffer, which all staging waves of a sweep wave count up),
// never at a barrier, and the sweep wave looks at a counter one chunk (one tile) before
// it needs it.
//
// Rows beyond 64 go to further sweep waves; wave w+1 consumes the last row of
// wave w through an LDS seam row guarded by a progress counter and simply runs a
// few steps behind.  Lattices taller than the workgroup's sweep waves are
// processed band after band with the same seam mechanism.
//
// The arithmetic follows the CPU reference operation for operation
// (fast_rnnt/csrc/mutual_information_cpu.cu:89-121 forward, :179-252 backward,
// log-add from fast_rnnt/csrc/mutual_information.h:36-65); only exp/log come
// from the GPU's own units.
#include "common.hip.h"

namespace frnnt {
namespace {

constexpr int kMaxSweep = 4;           // sweep waves per workgroup
constexpr int kChunk = 8;              // steps per seam hand-over
constexpr int kTileSteps = 32;         // steps per staged tile
constexpr int kTilePitch = kTileSteps + 4;  // rows start 16-byte aligned and spread over the banks
constexpr int kTileElems = kWave * kTilePitch;
constexpr int kSeamPad = kChunk;        // slack on either side of a seam row, so that a whole
                                       // chunk of seam values is written without bounds tests
// The slack on the left is a little longer: the last lane's chunk that starts at step e0
// (a multiple of kChunk) goes to seam columns e0 - 63 ..., and with 11 elements of slack
// their address is a multiple of 16 bytes, so that a chunk is two 16-byte LDS writes.
constexpr int kSeamPadLeft = kSeamPad + 3;
static_assert((kSeamPadLeft - (kWave - 1)) % 4 == 0, "seam chunks are not 16-byte aligned");
constexpr int kSeamSlack = kSeamPadLeft + kSeamPad;
constexpr int kFwdStagers = 3;         // staging waves per sweep wave
constexpr int kBwdStagers = 3;
// With at most two sweep waves a workgroup has room for more staging waves per sweep wave.
// The backward kernel's evaluate d1 / d2 and are what its sweep waves wait for (c2 shape:
// 17.2 us with 6, 16.9 with 7: 16 waves, the most a workgroup holds); the forward kernel's
// only copy (18.45 us with 2, 18.05 with 3, 17.9 with 4).
constexpr int kFwdStagersFew = 4;
constexpr int kBwdStagersFew = 7;
constexpr int kSpinLimit = 1 << 22;   // polls before a wait gives up (seconds, not microseconds)
// Set by frnnt_set_spin_limit(): lets a test force the give-up path from the host.
int g_spin_limit = kSpinLimit;

struct Window {
  int s0, t0, ns, nt;  // origin and extent (ns = s_end - s_begin, ...)
  bool ok;
};
// `checks` bits and `status[0]` codes of the forward kernel (FRNNT_CHECK_* / FRNNT_STATUS_*
// of the public header)
constexpr int kCheckSymbols = 1, kCheckFrames = 2;
constexpr int kStatusWindow = 1, kStatusNoSymbols = 2, kStatusFewFrames = 3;

__device__ __forceinline__ Window load_window(const int64_t *boundary, int b, int S, int T) {
  Window w{0, 0, S, T, true};
  if (boundary) {
    const int64_t a = boundary[4 * b + 0], c = boundary[4 * b + 1];
    const int64_t d = boundary[4 * b + 2], e = boundary[4 * b + 3];
    w.ok = (0 <= a) && (a <= d) && (d <= S) && (0 <= c) && (c <= e) && (e <= T);
    w.s0 = (int)a;
    w.t0 = (int)c;
    w.ns = (int)(d - a);
    w.nt = (int)(e - c);
  }
  return w;
}

// Blocks until the counter reaches `target`; gives up (returns false) after a
// bounded number of polls so that no wave can spin forever.
// A wave that gives up must not leave quietly: the callers mark the utterance's outputs
// (see give_up below), so that a wait that never ends shows as NaN, not as a wrong number.
__device__ __forceinline__ bool wait_for(const int *counter, int target, int limit) {
  int spins = 0;
  while (__hip_atomic_load(counter, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) < target) {
    __builtin_amdgcn_s_sleep(1);
    if (++spins > limit) return false;
  }
  return true;
}
// Non-blocking look at a counter: the value is used a chunk or a tile later, when it
// has long arrived.  LDS serves the reads of one wave in order, so data read after
// the counter is at least as recent as the counter; the empty asm keeps the compiler
// from moving such reads ahead of it.
__device__ __forceinline__ int peek(const int *counter) {
  const int v = __hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  asm volatile("" ::: "memory");
  return v;
}
// Waits until this wave's LDS reads have arrived.  On the rare path that re-reads the seam
// it keeps the common path's wait at "the read issued a chunk ago", which the LDS writes
// issued since then do not hold up (after a join the compiler takes the stricter wait).
__device__ __forceinline__ void lds_reads_done() {
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0) only
}
__device__ __forceinline__ void count_in(int *counter) {
  __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ void publish(int *counter, int value) {
  __hip_atomic_store(counter, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
}
// The same for a counter that only tells of LDS writes by this very wave: LDS carries
// out one wave's instructions in the order they were issued, so the counter's write
// lands after the data without the wave waiting for its writes to finish (a release
// makes it wait, ~190 cycles every time).  The empty asm keeps the compiler from
// moving the data's writes below the counter's.
__device__ __forceinline__ void publish_lds_writes(int *counter, int value) {
  asm volatile("" ::: "memory");
  __hip_atomic_store(counter, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  asm volatile("" ::: "memory");
}

// log(exp(a) + exp(c)) on the serial chain: same operation order as log_add(),
// written so that the only fix-up is the NaN that (-inf) - (-inf) produces.
__device__ __forceinline__ float chain_log_add(float a, float c) {
  const float d = a - c;
  const float hi = fmaxf(a, c);  // neither operand is ever NaN
  // -|d| * log2(e) is <= 0 or NaN ((-inf) - (-inf)); fminf maps the NaN to 0, and
  // the result is then hi + log(2) = hi, because hi is infinite in that case --
  // exactly the "return the larger operand" rule of the reference, without a branch.
  const float t = fminf(-fabsf(d) * 1.44269504088896341f, 0.0f);
  const float e = __builtin_amdgcn_exp2f(t);
  return __builtin_fmaf(__builtin_amdgcn_logf(1.0f + e), 0.693147180559945309f, hi);
}
__device__ __forceinline__ double chain_log_add(double a, double c) { return log_add(a, c); }

// Results go to memory through raw buffer stores: the resource covers one
// utterance's array, a lane passes a byte offset, and an offset of kDropped lies
// outside every resource, so the hardware's range check discards the store.  That
// turns "this lane has nothing to write here" into one select on the offset, with
// no branch and no change of the execution mask.
constexpr int kDropped = (int)0x80000000;
typedef int intx2 __attribute__((ext_vector_type(2)));
typedef int intx4 __attribute__((ext_vector_type(4)));

template <typename R>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t buffer_of(R *base, size_t elems) {
  // raw buffer (stride 0), 32-bit elements as far as the descriptor is concerned
  return __builtin_amdgcn_make_buffer_rsrc(base, 0, (int)(elems * sizeof(R)), 0x00020000);
}
__device__ __forceinline__ void put1(__amdgpu_buffer_rsrc_t rs, int off, float v) {
  __builtin_amdgcn_raw_buffer_store_b32(__float_as_int(v), rs, off, 0, 0);
}
__device__ __forceinline__ void put1(__amdgpu_buffer_rsrc_t rs, int off, double v) {
  const long long bits = __double_as_longlong(v);
  __builtin_amdgcn_raw_buffer_store_b64(intx2{(int)bits, (int)(bits >> 32)}, rs, off, 0, 0);
}
// Range-checked load: an offset outside the resource (negative ones included, they are
// huge when read as unsigned) reads as 0 and touches no memory.
__device__ __forceinline__ float get1(__amdgpu_buffer_rsrc_t rs, int off, float) {
  return __int_as_float(__builtin_amdgcn_raw_buffer_load_b32(rs, off, 0, 0));
}
__device__ __forceinline__ double get1(__amdgpu_buffer_rsrc_t rs, int off, double) {
  const intx2 v = __builtin_amdgcn_raw_buffer_load_b64(rs, off, 0, 0);
  return __longlong_as_double(((long long)v[1] << 32) | (unsigned int)v[0]);
}
// four consecutive elements (the address only needs element alignment)
__device__ __forceinline__ void put4(__amdgpu_buffer_rsrc_t rs, int off, float a, float b, float c,
                                     float d) {
  __builtin_amdgcn_raw_buffer_store_b128(
      intx4{__float_as_int(a), __float_as_int(b), __float_as_int(c), __float_as_int(d)}, rs, off,
      0, 0);
}
__device__ __forceinline__ void put4(__amdgpu_buffer_rsrc_t rs, int off, double a, double b,
                                     double c, double d) {
  const long long ab = __double_as_longlong(a), bb = __double_as_longlong(b);
  const long long cb = __double_as_longlong(c), db = __double_as_longlong(d);
  __builtin_amdgcn_raw_buffer_store_b128(
      intx4{(int)ab, (int)(ab >> 32), (int)bb, (int)(bb >> 32)}, rs, off, 0, 0);
  __builtin_amdgcn_raw_buffer_store_b128(
      intx4{(int)cb, (int)(cb >> 32), (int)db, (int)(db >> 32)}, rs, off == kDropped ? off : off + 16,
      0, 0);
}
// One lane's kTileSteps staged values, 16 bytes per LDS read.
template <typename R>
__device__ __forceinline__ void pull_row(R (&dst)[kTileSteps], const R *src) {
  constexpr int kPer = 16 / (int)sizeof(R);
  typedef R Piece __attribute__((ext_vector_type(kPer)));
  const Piece *s = reinterpret_cast<const Piece *>(src);
#pragma unroll
  for (int i = 0; i < kTileSteps / kPer; ++i) {
    const Piece v = s[i];
#pragma unroll
    for (int e = 0; e < kPer; ++e) dst[i * kPer + e] = v[e];
  }
}

// kChunk values of one lane into its tile row, 16 bytes per LDS write.
template <typename R>
__device__ __forceinline__ void push_chunk(R *dst, const R (&src)[kChunk]) {
  constexpr int kPer = 16 / (int)sizeof(R);
  typedef R Piece __attribute__((ext_vector_type(kPer)));
  Piece *d = reinterpret_cast<Piece *>(dst);
#pragma unroll
  for (int i = 0; i < kChunk / kPer; ++i) {
    Piece v;
#pragma unroll
    for (int e = 0; e < kPer; ++e) v[e] = src[i * kPer + e];
    d[i] = v;
  }
}

// The first (kHalf = 0) or second half of a chunk into its place in the tile row.  An LDS
// write takes its data out of the registers over some 30 cycles after it has been issued,
// and an instruction that overwrites one of them waits for that; so a sweep wave writes
// the first half of a chunk as soon as it is complete, in the middle of the chunk, and
// the second half at its end: each half then has four steps' time before the next chunk
// comes to its registers.
template <int kHalf, typename R>
__device__ __forceinline__ void push_half(R *dst, const R (&src)[kChunk]) {
  constexpr int kPer = 16 / (int)sizeof(R);
  typedef R Piece __attribute__((ext_vector_type(kPer)));
  Piece *d = reinterpret_cast<Piece *>(dst);
#pragma unroll
  for (int i = kHalf * (kChunk / 2 / kPer); i < (kHalf + 1) * (kChunk / 2 / kPer); ++i) {
    Piece v;
#pragma unroll
    for (int e = 0; e < kPer; ++e) v[e] = src[i * kPer + e];
    d[i] = v;
  }
}

// Keeps the registers of a half chunk that has just been written to LDS from being given
// to the next results at once (see push_half): called four steps later, it makes them
// count as still in use until then.  Emits no instruction.
template <typename R>
__device__ __forceinline__ void still_in_use(const R (&v)[kChunk], int first) {
  if constexpr (sizeof(R) == 4) {
    asm volatile("" ::"v"(v[first]), "v"(v[first + 1]), "v"(v[first + 2]), "v"(v[first + 3]));
  }
}

struct Counters {
  int failed;                             // set by a wave whose bounded wait ran out
  int ready[kMaxSweep];                   // seam columns published by sweep wave w
  int written[kMaxSweep];                 // tiles whose results sweep wave w has left in LDS
  // per sweep wave w and tile buffer k (index w * buffers + k): how many times a staging
  // wave has finished staging a tile into that buffer, all of w's staging waves and all
  // tiles together -- the buffer's n-th tile is complete at n * stagers.  One counter for
  // all staging waves: a sweep wave pays for every test it makes.
  int loaded[16];
};

// Geometry of what sweep wave `w` does in band `band`; identical on the sweep
// wave and on its staging waves.
struct Band {
  int row0, nrows, nsteps, ntiles;
};
__device__ __forceinline__ Band band_of(int band, int w, int nsweep, int NS, int NT) {
  Band g;
  g.row0 = (band * nsweep + w) * kWave;
  g.nrows = min(kWave, NS + 1 - g.row0);
  g.nsteps = NT + g.nrows;
  g.ntiles = (g.nsteps + kTileSteps - 1) / kTileSteps;
  return g;
}

// The tiles [lo, hi) of a sweep wave's band that are plain: all 32 steps exist
// ((m + 1) * 32 <= nsteps), the step that holds the wave's result (fin_step, if any) is not
// among them and, for a wave with a seam above it, every seam column that the tile and the
// first chunk after it look at exists (0 <= 32 m - shift, 32 (m + 1) + 7 - shift <= NT).
struct PlainTiles {
  int lo, hi;
};
__device__ __forceinline__ PlainTiles plain_tiles(const Band &g, int fin_step, bool up, int shift, int NT) {
  PlainTiles t;
  t.lo = (up && shift > 0) ? 1 : 0;
  t.hi = g.nsteps / kTileSteps;
  if (fin_step >= 0) t.hi = min(t.hi, fin_step / kTileSteps);
  if (up) t.hi = min(t.hi, max(NT - (kChunk - 1) + shift, 0) / kTileSteps);
  t.lo = min(t.lo, g.ntiles);
  t.hi = max(min(t.hi, g.ntiles), t.lo);
  return t;
}

// =============================== forward =====================================
// Staged per step and row: x = px feeding the cell from the row below,
// y = py feeding it from the left; -inf where that edge does not exist, and
// y = 0 at the origin cell so that the chain produces p = 0 there.
// A sweep wave only runs the chain: it takes a tile's x / y from an LDS buffer and
// leaves the tile's p in the place of x (16 bytes per LDS write); the staging waves
// carry p to memory, each for the rows it stages, before they refill the buffer.
// kSweepCap: most sweep waves the launch may use; it only sets the register budget.
template <typename R, bool kModified, int kSweepCap, int kStagers, int kBuffers>
__global__ void __launch_bounds__((1 + kStagers) * kSweepCap *kWave)
    mi_forward_kernel(const R *__restrict__ px, const R *__restrict__ py,
                      const int64_t *__restrict__ boundary, R *__restrict__ p,
                      R *__restrict__ ans, int S, int T, int spin_limit, int checks,
                      int *__restrict__ status) {
  extern __shared__ __align__(16) unsigned char dyn_lds[];
  __shared__ Counters cnt;

  const int b = blockIdx.x;
  const int nsweep = blockDim.x / (kWave * (1 + kStagers));
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);  // in a scalar register
  const int lane = threadIdx.x % kWave;
  const int T1 = kModified ? T : T + 1;
  const int TP = T + 1;
  const int shift = kModified ? 1 : 0;
  const R ninf = Num<R>::neg_inf();

  const Window win = load_window(boundary, b, S, T);
  // What the loss functions assert of a boundary row before they call the recursion
  // (rnnt_loss.py:25-42), for callers that do not want to wait for a host copy of the rows:
  // a row that fails is treated like one whose window is out of range, and `status` -- memory
  // the host can read, e.g. pinned host memory -- names the failed test and the row.
  int bad = win.ok ? 0 : kStatusWindow;
  if (checks != 0 && boundary != nullptr && win.ok) {
    if ((checks & kCheckSymbols) && win.s0 + win.ns < 1) bad = kStatusNoSymbols;
    else if ((checks & kCheckFrames) && win.t0 + win.nt < win.s0 + win.ns) bad = kStatusFewFrames;
  }
  if (bad != 0) {
    if (threadIdx.x == 0) {
      ans[b] = std::numeric_limits<R>::quiet_NaN();
      if (status) {
        status[1] = b;
        status[0] = bad;
      }
    }
    return;
  }
  if (threadIdx.x < (int)(sizeof(Counters) / sizeof(int)))
    reinterpret_cast<int *>(&cnt)[threadIdx.x] = 0;
  __syncthreads();

  const int NS = win.ns, NT = win.nt, cols = NT + 1;
  const R *pxb = px + (size_t)b * S * T1;
  const R *pyb = py + (size_t)b * (S + 1) * T;
  R *pb = p + (size_t)b * (S + 1) * TP;
  R *seam = reinterpret_cast<R *>(dyn_lds);
  const int seam_pitch = (TP + kSeamSlack + 3) & ~3;  // keeps the tiles 16-byte aligned
  R *tiles = seam + (size_t)nsweep * seam_pitch;  // per sweep wave: kBuffers x tiles, then as many y tiles
  const int band_rows = kWave * nsweep;
  // A wave whose bounded wait ran out: the utterance's score becomes NaN (also for the
  // wave that would store it later), so the failure cannot pass for a result.
  auto give_up = [&]() {
    if (lane == 0) {
      publish(&cnt.failed, 1);
      ans[b] = std::numeric_limits<R>::quiet_NaN();
    }
  };

  if (wave >= nsweep) {
    // ------------------------------ staging wave -------------------------------
    const int w = (wave - nsweep) / kStagers, l = (wave - nsweep) % kStagers;
    R *base = tiles + (size_t)w * 2 * kBuffers * kTileElems;
    const int half = lane >> 5, q = lane & 31;
    // rows of a tile this wave stages: r(u) = 2*l + half + 2*kStagers*u
    constexpr int kRows = (kWave + 2 * kStagers - 1) / (2 * kStagers);
    struct Staged {
      R x[kRows], y[kRows];
    };
    // Global fetches of tile m+1 are issued (into registers) as soon as tile m is staged,
    // before this wave waits for the next LDS buffer, so their latency overlaps the
    // sweep.  The loads are range-checked and otherwise unconditional: what a lane reads
    // for cells outside the window is either replaced at staging time (row 0, column 0:
    // the -inf that closes the lattice) or never reaches a cell of the window (columns
    // before a row's start or beyond its end only feed cells at least as far out).
    const __amdgpu_buffer_rsrc_t px_rsrc = buffer_of(const_cast<R *>(pxb), (size_t)S * T1);
    const __amdgpu_buffer_rsrc_t py_rsrc = buffer_of(const_cast<R *>(pyb), (size_t)(S + 1) * T);
    const __amdgpu_buffer_rsrc_t p_rsrc = buffer_of(pb, (size_t)(S + 1) * TP);
    constexpr int kStep = 2 * kStagers;
    constexpr int kSize = (int)sizeof(R);
    const int r_first = 2 * l + half;
    auto fetch = [&](Staged &in, const Band &g, int m) {
      const int s_first = win.s0 + g.row0 + r_first;
      const int j_first = m * kTileSteps + q - r_first;
      const int x0 = ((s_first - 1) * T1 + win.t0 + j_first - shift) * kSize;
      const int y0 = (s_first * T + win.t0 + j_first - 1) * kSize;
#pragma unroll
      for (int u = 0; u < kRows; ++u) {
        // kStep rows further up: as many rows down in memory, as many columns left
        in.x[u] = get1(px_rsrc, x0 + u * (kStep * (T1 - 1) * kSize), R());
        in.y[u] = get1(py_rsrc, y0 + u * (kStep * (T - 1) * kSize), R());
      }
    };
    // p of tile pm of the band that starts at row0, left by the sweep wave in buffer `buf`:
    // element (row r, step q) is the cell (row0 + r, 32 pm + q - r) of the window.  Taking
    // it out of the buffer and storing it are two steps: a wave's wait for a load also
    // waits for every store it has issued before, so the stores of a tile go out after
    // the buffer has been refilled and handed back to the sweep wave, not before.
    struct Drained {
      R v[kRows];
      int row0, pm;
    };
    auto take = [&](Drained &d, int row0, int pm, int buf) {
      const R *ps = base + buf * kTileElems + r_first * kTilePitch + q;
      d.row0 = row0;
      d.pm = pm;
#pragma unroll
      for (int u = 0; u < kRows; ++u) {
        if (r_first + kStep * u >= kWave) continue;
        d.v[u] = ps[u * kStep * kTilePitch];
      }
    };
    auto store = [&](const Drained &d) {
      const int i0 = d.row0 + r_first;
      const int j0 = d.pm * kTileSteps + q - r_first;
      const int o0 = ((win.s0 + i0) * TP + win.t0 + j0) * kSize;
#pragma unroll
      for (int u = 0; u < kRows; ++u) {
        if (r_first + kStep * u >= kWave) continue;
        const int i = i0 + kStep * u, j = j0 - kStep * u;
        const bool ok = i <= NS && (unsigned)j <= (unsigned)NT;
        put1(p_rsrc, ok ? o0 + u * (kStep * (TP - 1) * kSize) : kDropped, d.v[u]);
      }
    };
    // which tile each buffer holds: its band's first row and its number in the band
    int held_row0[kBuffers], held_m[kBuffers];
#pragma unroll
    for (int k = 0; k < kBuffers; ++k) held_row0[k] = held_m[k] = 0;
    auto take_buffer = [&](Drained &d, int buf) {
      int row0 = held_row0[0], pm = held_m[0];
#pragma unroll
      for (int k = 1; k < kBuffers; ++k) {
        row0 = buf == k ? held_row0[k] : row0;
        pm = buf == k ? held_m[k] : pm;
      }
      take(d, row0, pm, buf);
    };
    int tile_base = 0, buf = 0;  // buf = tile number modulo kBuffers
    for (int band = 0; band * band_rows <= NS; ++band) {
      const Band g = band_of(band, w, nsweep, NS, NT);
      if (g.row0 > NS) break;
      Staged cur;
      fetch(cur, g, 0);
      for (int m = 0; m < g.ntiles; ++m) {
        const int gt = tile_base + m;
        Drained out;
        const bool refill = gt >= kBuffers;
        if (refill) {
          // the buffer still holds p of tile gt - kBuffers
          if (!wait_for(&cnt.written[w], gt - kBuffers + 1, spin_limit)) {
            give_up();
            return;
          }
          take_buffer(out, buf);
        }
#pragma unroll
        for (int k = 0; k < kBuffers; ++k) {
          held_row0[k] = buf == k ? g.row0 : held_row0[k];
          held_m[k] = buf == k ? m : held_m[k];
        }
        R *xdst = base + buf * kTileElems + r_first * kTilePitch + q;
        R *ydst = xdst + kBuffers * kTileElems;
        // only the first tiles hold a column 0 (local step = row), and only the first
        // band holds row 0
        const bool starts = m * kTileSteps <= kWave - 1 + shift;
#pragma unroll
        for (int u = 0; u < kRows; ++u) {
          const int r = r_first + kStep * u;
          if (r >= kWave) continue;
          R x = cur.x[u], y = cur.y[u];
          const int i = g.row0 + r;
          if (starts) {
            const int j = m * kTileSteps + q - r;
            if (j <= 0) y = (j == 0 && i == 0) ? (R)0 : ninf;
            if (j < shift) x = ninf;
          }
          if (u == 0 && i == 0) x = ninf;
          xdst[u * kStep * kTilePitch] = x;
          ydst[u * kStep * kTilePitch] = y;
        }
        // every lane's LDS writes precede the release by lane 0 of the same wave
        if (lane == 0) count_in(&cnt.loaded[w * kBuffers + buf]);
        if (refill) store(out);
        // the next tile's inputs, fetched while this wave waits for its buffer
        if (m + 1 < g.ntiles) fetch(cur, g, m + 1);
        buf = buf + 1 == kBuffers ? 0 : buf + 1;
      }
      tile_base += g.ntiles;
    }
    // the tiles still in the buffers
    const int first_left = max(tile_base - kBuffers, 0);
    buf = first_left % kBuffers;
    for (int gt = first_left; gt < tile_base; ++gt) {
      if (!wait_for(&cnt.written[w], gt + 1, spin_limit)) {
        give_up();
        return;
      }
      Drained out;
      take_buffer(out, buf);
      store(out);
      buf = buf + 1 == kBuffers ? 0 : buf + 1;
    }
    return;
  }

  // -------------------------------- sweep wave ---------------------------------
  const int w = wave;
  const int prev = (w + nsweep - 1) % nsweep;
  R *my_seam = seam + (size_t)w * seam_pitch + kSeamPadLeft;
  const R *up_seam = seam + (size_t)prev * seam_pitch + kSeamPadLeft;
  R *base = tiles + (size_t)w * 2 * kBuffers * kTileElems;
  int tile_base = 0, buf = 0, rounds = 0;  // tile number modulo kBuffers, and divided by it
  for (int band = 0; band * band_rows <= NS; ++band) {
    const Band g = band_of(band, w, nsweep, NS, NT);
    if (g.row0 > NS) break;
    const int i = g.row0 + lane;
    const bool has_up = g.row0 > 0;
    const int up_base = (w > 0 ? band : band - 1) * cols;
    const int my_base = band * cols;
    // the answer is the cell (NS, NT): lane NS - row0 at step NT + NS - row0
    const int fin_lane = NS - g.row0;
    const int fin_step = (fin_lane < kWave) ? NT + fin_lane : -1;

    R own = (i == 0) ? (R)0 : ninf, own2 = ninf;
    R fin = ninf;
    const R *seam_at = up_seam + (lane - shift);  // seam_at[e]: what lane 0 needs at step e + lane
    const bool has_down = g.row0 + kWave <= NS;  // rows below this wave's: someone reads the seam
    // counters and seam values are read one chunk (one tile) ahead of their use, so
    // that the LDS round trip is off the chain; a stale value only costs a re-read
    int seen_ready = 0;
    R seen_seam = ninf;
    int seen_loaded = 0;
    // One tile, specialised at compile time on whether the wave receives a seam (kUp),
    // feeds one (kDown), and on kPlain: a tile whose 32 steps all exist, do not hold the
    // answer's step and, with a seam above, look at existing seam columns only.  A single
    // wave pays for every instruction it issues, scalar tests and branches included, so
    // plain tiles run without the tests; and every kind of tile has a loop of its own (see
    // sweep_tiles): with all kinds in one loop body the compiler's code for the steps
    // themselves took twice as long.
    auto one_tile = [&](int m, auto up_c, auto down_c, auto plain_c) __attribute__((always_inline)) -> bool {
      constexpr bool kUp = decltype(up_c)::value;
      constexpr bool kDown = decltype(down_c)::value;
      constexpr bool kPlain = decltype(plain_c)::value;
      const int gt = tile_base + m;
      if (__builtin_amdgcn_readfirstlane(seen_loaded) < kStagers * (rounds + 1) &&
          !wait_for(&cnt.loaded[w * kBuffers + buf], kStagers * (rounds + 1), spin_limit)) {
        give_up();
        return false;
      }
      // this lane's 32 steps of inputs go to registers in one burst
      R xq[kTileSteps], yq[kTileSteps];
      R *x_row = base + buf * kTileElems + lane * kTilePitch;  // x in, p out
      pull_row(xq, x_row);
      pull_row(yq, x_row + kBuffers * kTileElems);
      buf = buf + 1 == kBuffers ? 0 : buf + 1;
      rounds += buf == 0;

      bool failed = false;
      R last[kChunk];  // the chunk before
#pragma unroll
      for (int k = 0; k < kChunk; ++k) last[k] = 0;
      // one chunk of kChunk steps
      auto chunk = [&](int c4, int e0) __attribute__((always_inline)) {
        R handed = ninf;  // lane k: the seam value lane 0 needs at step e0 + k
        if (kUp) {
          const int need = kPlain ? e0 + kChunk - shift : min(e0 + kChunk - shift, cols);
          handed = seen_seam;
          if ((kPlain || need > 0) && __builtin_amdgcn_readfirstlane(seen_ready) < up_base + need) {
            // (a wait that has run out is not tried again: the wave finishes its tile on
            // whatever the seam holds and then gives up)
            if (!failed && !wait_for(&cnt.ready[prev], up_base + need, spin_limit)) failed = true;
            const int col = e0 + lane - shift;
            handed = (lane < kChunk && col >= 0 && col <= NT) ? up_seam[col] : ninf;
            lds_reads_done();
          }
          // next chunk's counter, then its seam values (LDS serves a wave in order)
          seen_ready = peek(&cnt.ready[prev]);
          if (kPlain) {
            // every column this tile and the first chunk after it look at exists: no
            // tests, and what lanes 8 .. 63 read never reaches lane 0
            seen_seam = seam_at[e0 + kChunk];
          } else {
            const int col = e0 + kChunk + lane - shift;
            seen_seam = ninf;
            if (lane < kChunk && col >= 0 && col <= NT) seen_seam = up_seam[col];
          }
          // (the reads above are for the next chunk: they are issued here, before the steps)
          __builtin_amdgcn_sched_barrier(0);
        }
        if (c4 == kTileSteps / kChunk - 1) seen_loaded = peek(&cnt.loaded[w * kBuffers + buf]);
        R vals[kChunk];
#pragma unroll
        for (int k = 0; k < kChunk; ++k) {
          const int kk = c4 * kChunk + k;
          // lane 0 of a wave without a seam owns lattice row 0, whose x is -inf,
          // so the 0 it receives from the shift never matters
          R up;
          if (kUp) {
            // lane 0 takes the seam value of this step, which then moves on
            up = from_lane_below_or(kModified ? own2 : own, handed);
            handed = from_lane_above(handed);
          } else {
            up = from_lane_below_zero(kModified ? own2 : own);
          }
          const R v = chain_log_add(up + xq[kk], own + yq[kk]);
          vals[k] = v;
          own2 = own;
          own = v;
          if (k == kChunk / 2 - 1) {
            // the chunk's p takes the place of its x in the tile: first half
            push_half<0>(x_row + c4 * kChunk, vals);
            still_in_use(last, kChunk / 2);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
        still_in_use(vals, 0);
        if (!kPlain) {
          const int kf = fin_step - e0;  // wave-uniform
          if ((unsigned)kf < (unsigned)kChunk) {
#pragma unroll
            for (int k = 0; k < kChunk; ++k)
              if (k == kf) fin = vals[k];
          }
        }
        // seam: the last lane's columns e0 - 63 ... (the pads take what falls outside)
        if (kDown && e0 + kChunk > kWave - 1) {
          if (lane == kWave - 1) {
            push_chunk(my_seam + (e0 - (kWave - 1)), vals);
            const int done = max(0, min(e0 + kChunk - (kWave - 1), cols));
            publish_lds_writes(&cnt.ready[w], my_base + done);
          }
        }
        push_half<1>(x_row + c4 * kChunk, vals);
#pragma unroll
        for (int k = kChunk / 2; k < kChunk; ++k) last[k] = vals[k];
      };
#pragma unroll
      for (int c4 = 0; c4 < kTileSteps / kChunk; ++c4) {
        const int e0 = m * kTileSteps + c4 * kChunk;
        if (kPlain || e0 < g.nsteps) chunk(c4, e0);
      }
      if (failed) {
        give_up();
        return false;
      }
      if (lane == 0) publish_lds_writes(&cnt.written[w], gt + 1);
      return true;
    };
    // the band's tiles: those before the plain ones, the plain ones, the rest
    auto sweep_tiles = [&](auto up_c, auto down_c) __attribute__((always_inline)) -> bool {
      const PlainTiles plain = plain_tiles(g, fin_step, decltype(up_c)::value, shift, NT);
      for (int m = 0; m < plain.lo; ++m)
        if (!one_tile(m, up_c, down_c, std::false_type{})) return false;
      for (int m = plain.lo; m < plain.hi; ++m)
        if (!one_tile(m, up_c, down_c, std::true_type{})) return false;
      for (int m = plain.hi; m < g.ntiles; ++m)
        if (!one_tile(m, up_c, down_c, std::false_type{})) return false;
      return true;
    };
    bool done;
    if (has_up)
      done = has_down ? sweep_tiles(std::true_type{}, std::true_type{})
                      : sweep_tiles(std::true_type{}, std::false_type{});
    else
      done = has_down ? sweep_tiles(std::false_type{}, std::true_type{})
                      : sweep_tiles(std::false_type{}, std::false_type{});
    if (!done) return;
    if (lane == fin_lane) {
      ans[b] = peek(&cnt.failed) ? std::numeric_limits<R>::quiet_NaN() : fin;
      // A staging wave may give up between that look and the store, and its NaN must not be
      // covered by the score: once the store has left, look again.  A wave that gives up
      // after this second look stores its NaN after it, and so after the score.
      __threadfence();
      if (__hip_atomic_load(&cnt.failed, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP))
        ans[b] = std::numeric_limits<R>::quiet_NaN();
    }
    tile_base += g.ntiles;
  }
}

// =============================== backward ====================================
// Rows and columns are counted from the end of the window (r = NS - i,
// c = NT - j); lane L of a sweep wave owns reversed row r and works on reversed
// column e - L at local step e.  A cell's gradient is what the row above hands
// down plus what its right neighbour hands left; it is then split into a d1
// share for the cell below and a d2 share for the cell to the left.  The staging
// waves evaluate d1 / d2 (mutual_information_cpu.cu:196-212 and the two edge
// loops :219-235).  A single wave issues one instruction every 4-5 cycles, and a sweep
// wave that also computes addresses and stores its results spends ~140 cycles per
// step where the dependent chain (shift, add, multiply) needs ~25; so the sweep wave
// only leaves the px / py gradients of a tile in the LDS buffer it has just read that
// tile's d1 / d2 from (a lane's 32 steps, 16 bytes per write), and the staging waves
// carry them to memory, each for the rows it stages, before they refill the buffer.
template <typename R, bool kModified, int kSweepCap, int kStagers, int kBuffers>
__global__ void __launch_bounds__((1 + kStagers) * kSweepCap *kWave)
    mi_backward_kernel(const R *__restrict__ px, const int64_t *__restrict__ boundary,
                       const R *__restrict__ p, R *ans_grad, R *__restrict__ px_grad,
                       R *__restrict__ py_grad, int S, int T, int overwrite_ans_grad,
                       const R *__restrict__ scores, R *__restrict__ loss, int B, int reduction,
                       int spin_limit) {
  extern __shared__ __align__(16) unsigned char dyn_lds[];
  __shared__ Counters cnt;

  const int b = blockIdx.x;
  const int nsweep = blockDim.x / (kWave * (1 + kStagers));
  const int nwaves = blockDim.x / kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);  // in a scalar register
  const int lane = threadIdx.x % kWave;
  const int T1 = kModified ? T : T + 1;
  const int TP = T + 1;
  const int shift = kModified ? 1 : 0;

  const Window win = load_window(boundary, b, S, T);
  R *gxb = px_grad + (size_t)b * S * T1;
  R *gyb = py_grad + (size_t)b * (S + 1) * T;
  const __amdgpu_buffer_rsrc_t gx_rsrc = buffer_of(gxb, (size_t)S * T1);
  const __amdgpu_buffer_rsrc_t gy_rsrc = buffer_of(gyb, (size_t)(S + 1) * T);

  // Exact zeros everywhere the sweep does not write, one wave per row.  The staging
  // waves do this once they are two tiles ahead of their sweep wave, off the critical
  // path (a barrier after these stores would have to wait until they have all reached
  // memory).
  // elements [begin, end) of the row that starts at element `row` of the resource;
  // begin and end are wave-uniform
  auto zero_range = [&](__amdgpu_buffer_rsrc_t rs, int row, int begin, int end) {
    const int len = end - begin;
    if (len <= 0) return;
    const R z = 0;
    if (len < 4) {
      put1(rs, lane < len ? (row + begin + lane) * (int)sizeof(R) : kDropped, z);
      return;
    }
    for (int t0 = begin; t0 + 4 <= end; t0 += 4 * kWave) {
      const int t = t0 + 4 * lane;
      put4(rs, t + 4 <= end ? (row + t) * (int)sizeof(R) : kDropped, z, z, z, z);
    }
    // what is left of the last group, as one group that ends with the range
    if (len & 3) put4(rs, lane == 0 ? (row + end - 4) * (int)sizeof(R) : kDropped, z, z, z, z);
  };
  auto zero_outside = [&](int part, int parts) {
    if (!boundary) return;
    const int s_lo = win.s0, s_hi = win.s0 + win.ns;
    const int t_lo = win.t0, t_hi = win.t0 + win.nt;
    for (int s = part; s <= S; s += parts) {
      if (s < S) {
        if (win.ok && s >= s_lo && s < s_hi) {
          zero_range(gx_rsrc, s * T1, 0, t_lo);
          zero_range(gx_rsrc, s * T1, t_hi - shift + 1, T1);
        } else {
          zero_range(gx_rsrc, s * T1, 0, T1);
        }
      }
      if (win.ok && s >= s_lo && s <= s_hi) {
        zero_range(gy_rsrc, s * T, 0, t_lo);
        zero_range(gy_rsrc, s * T, t_hi, T);
      } else {
        zero_range(gy_rsrc, s * T, 0, T);
      }
    }
  };
  if (!win.ok) {
    zero_outside(wave, nwaves);
    if (loss && b == 0 && wave == 0) reduce_scores(scores, loss, B, reduction, lane);
    return;
  }
  if (threadIdx.x < (int)(sizeof(Counters) / sizeof(int)))
    reinterpret_cast<int *>(&cnt)[threadIdx.x] = 0;
  __syncthreads();

  const int NS = win.ns, NT = win.nt, cols = NT + 1;
  const R *pxb = px + (size_t)b * S * T1;
  const R *pb = p + (size_t)b * (S + 1) * TP;
  R *seam = reinterpret_cast<R *>(dyn_lds);
  const int seam_pitch = (TP + kSeamSlack + 3) & ~3;  // keeps the tiles 16-byte aligned
  R *tiles = seam + (size_t)nsweep * seam_pitch;  // per sweep wave: kBuffers d1 tiles, then as many d2 tiles
  const int band_rows = kWave * nsweep;
  // A wave whose bounded wait ran out leaves NaN where the window starts -- in px_grad,
  // in py_grad and, when it is written back, in ans_grad -- so that the utterance's
  // gradients cannot pass for a result; every staging wave repeats that when it is done
  // and finds the mark, so no later store of a good value covers it up.
  auto poison = [&]() {
    if (lane != 0) return;
    const R nan = std::numeric_limits<R>::quiet_NaN();
    if (NS > 0) put1(gx_rsrc, (win.s0 * T1 + win.t0) * (int)sizeof(R), nan);
    if (NT > 0) put1(gy_rsrc, (win.s0 * T + win.t0) * (int)sizeof(R), nan);
    if (overwrite_ans_grad && ans_grad) ans_grad[b] = nan;
  };
  auto give_up = [&]() {
    if (lane == 0) publish(&cnt.failed, 1);
    poison();
  };

  if (wave >= nsweep) {
    // ------------------------------ staging wave -------------------------------
    const int w = (wave - nsweep) / kStagers, l = (wave - nsweep) % kStagers;
    R *base = tiles + (size_t)w * 2 * kBuffers * kTileElems;
    const int half = lane >> 5, q = lane & 31;
    // rows of a tile this wave stages: r(u) = 2*l + half + 2*kStagers*u
    constexpr int kRows = (kWave + 2 * kStagers - 1) / (2 * kStagers);
    struct Staged {
      R here[kRows], below[kRows], x[kRows];
    };
    // Global fetches of tile m+1 are issued (into registers) as soon as tile m is staged,
    // before this wave waits for the next LDS buffer, so their latency overlaps the
    // sweep.  The loads are range-checked and otherwise unconditional; staging replaces
    // what was read for cells outside the window.
    const __amdgpu_buffer_rsrc_t p_rsrc = buffer_of(const_cast<R *>(pb), (size_t)(S + 1) * TP);
    const __amdgpu_buffer_rsrc_t px_rsrc = buffer_of(const_cast<R *>(pxb), (size_t)S * T1);
    constexpr int kStep = 2 * kStagers;
    constexpr int kSize = (int)sizeof(R);
    const int r_first = 2 * l + half;
    auto fetch = [&](Staged &in, const Band &g, int m) {
      // element offsets of row u = 0; each further u is kStep rows up the reversed
      // lattice, i.e. that many rows down in memory and as many columns right
      const int s_first = win.s0 + NS - (g.row0 + r_first);
      const int j_first = NT - (m * kTileSteps + q - r_first);
      const int below0 = ((s_first - 1) * TP + win.t0 + j_first - shift) * kSize;
      const int x0 = ((s_first - 1) * T1 + win.t0 + j_first - shift) * kSize;
      const int here0 = (s_first * TP + win.t0 + j_first) * kSize;
#pragma unroll
      for (int u = 0; u < kRows; ++u) {
        in.below[u] = get1(p_rsrc, below0 - u * (kStep * (TP - 1) * kSize), R());
        in.x[u] = get1(px_rsrc, x0 - u * (kStep * (T1 - 1) * kSize), R());
        in.here[u] = get1(p_rsrc, here0 - u * (kStep * (TP - 1) * kSize), R());
      }
    };
    // Gradients of tile m of band g, left by the sweep wave in buffer `buf`: element
    // (row r, step q) is the cell in reversed column c = 32 m + q - r, i.e. column
    // j = NT - c of lattice row i = NS - (row0 + r); gx goes to px_grad[s-1][t0 + j - shift],
    // gy to py_grad[s][t0 + j - 1], where those exist (mutual_information_cpu.cu:213-216).
    // The straight-line form below (every row group handled alike, borders by select) is
    // faster than variants that skip the rows past the window's top or branch to a
    // mask-free copy for tiles inside the window: those were 1 to 5 us slower per launch.
    // Taking a tile's gradients out of the buffer and storing them are two steps: a wave's
    // wait for a load also waits for every store it has issued before, so the stores go
    // out after the buffer has been refilled and handed back to the sweep wave.
    struct Drained {
      R vx[kRows], vy[kRows];
      int row0, pm;
    };
    auto take = [&](Drained &d, int pg_row0, int pm, int buf) {
      const R *gxs = base + buf * kTileElems + r_first * kTilePitch + q;
      const R *gys = gxs + kBuffers * kTileElems;
      d.row0 = pg_row0;
      d.pm = pm;
#pragma unroll
      for (int u = 0; u < kRows; ++u) {
        if (r_first + kStep * u >= kWave) continue;
        d.vx[u] = gxs[u * kStep * kTilePitch];
        d.vy[u] = gys[u * kStep * kTilePitch];
      }
    };
    auto store = [&](const Drained &d) {
      constexpr int kMinX = kModified ? 1 : 0;
      const int i0 = NS - d.row0 - r_first;                   // lattice row of u = 0
      const int j0 = NT - (d.pm * kTileSteps + q - r_first);  // and its column
      const int x0 = ((win.s0 + i0 - 1) * T1 + win.t0 - shift + j0) * kSize;
      const int y0 = ((win.s0 + i0) * T + win.t0 - 1 + j0) * kSize;
#pragma unroll
      for (int u = 0; u < kRows; ++u) {
        if (r_first + kStep * u >= kWave) continue;
        // one row group further: kStep rows up in memory and as many columns right
        const int xo = x0 - u * (kStep * (T1 - 1) * kSize), yo = y0 - u * (kStep * (T - 1) * kSize);
        const int i = i0 - kStep * u, j = j0 + kStep * u;
        const bool okx = i > 0 && (unsigned)(j - kMinX) < (unsigned)(NT + 1 - kMinX);
        const bool oky = i >= 0 && (unsigned)(j - 1) < (unsigned)NT;
        put1(gx_rsrc, okx ? xo : kDropped, d.vx[u]);
        put1(gy_rsrc, oky ? yo : kDropped, d.vy[u]);
      }
    };
    // which tile each buffer holds: its band's first row and its number in the band
    int held_row0[kBuffers], held_m[kBuffers];
#pragma unroll
    for (int k = 0; k < kBuffers; ++k) held_row0[k] = held_m[k] = 0;
    auto take_buffer = [&](Drained &d, int buf) {
      int row0 = held_row0[0], pm = held_m[0];
#pragma unroll
      for (int k = 1; k < kBuffers; ++k) {
        row0 = buf == k ? held_row0[k] : row0;
        pm = buf == k ? held_m[k] : pm;
      }
      take(d, row0, pm, buf);
    };
    int tile_base = 0, buf = 0;  // buf = tile number modulo kBuffers
    bool zeroed = false;
    for (int band = 0; band * band_rows <= NS; ++band) {
      const Band g = band_of(band, w, nsweep, NS, NT);
      if (g.row0 > NS) break;
      Staged cur;
      fetch(cur, g, 0);
      for (int m = 0; m < g.ntiles; ++m) {
        const int gt = tile_base + m;
        Drained out;
        const bool refill = gt >= kBuffers;
        if (refill) {
          // the buffer still holds the gradients of tile gt - kBuffers
          if (!wait_for(&cnt.written[w], gt - kBuffers + 1, spin_limit)) {
            give_up();
            return;
          }
          take_buffer(out, buf);
        }
#pragma unroll
        for (int k = 0; k < kBuffers; ++k) {
          held_row0[k] = buf == k ? g.row0 : held_row0[k];
          held_m[k] = buf == k ? m : held_m[k];
        }
        R *d1dst = base + buf * kTileElems + r_first * kTilePitch + q;
        R *d2dst = d1dst + kBuffers * kTileElems;
        // Only two borders of the window need care here.  Column 0 hands everything down
        // (mutual_information_cpu.cu:219-226; nothing at all in the modified lattice) and
        // the top row hands everything left (:228-235).  Everywhere else outside the
        // window the sweep needs no zeros: cells a row passes before its first column keep
        // a gradient of exactly 0 (nothing has reached them, and d1 / d2 are finite), and
        // what is computed past column 0 or above the top row only feeds cells further
        // out, none of which is stored or handed to another wave.
        const int at_col0 = NT - m * kTileSteps;  // q - r of the cells in column 0
        const int top_r = NS - g.row0;            // the top row, if it lies in this band
#pragma unroll
        for (int u = 0; u < kRows; ++u) {
          const int r = r_first + kStep * u;
          if (r >= kWave) continue;
          // mutual_information_cpu.cu:196-212
          const R term1 = cur.below[u] + cur.x[u];
          R total = cur.here[u];
          if (total - total != 0) total = 0;
          R d1 = Num<R>::exp_(term1 - total);
          R d2 = (R)1 - d1;
          if (d1 - d1 != 0) d1 = d2 = 0;
          if (q - r == at_col0) d1 = kModified ? (R)0 : (R)1;
          if (r == top_r) d2 = 1;
          d1dst[u * kStep * kTilePitch] = d1;
          d2dst[u * kStep * kTilePitch] = d2;
        }
        // every lane's LDS writes precede the release by lane 0 of the same wave
        if (lane == 0) count_in(&cnt.loaded[w * kBuffers + buf]);
        if (refill) store(out);
        // the next tile's inputs, fetched while this wave waits for its buffer
        if (m + 1 < g.ntiles) fetch(cur, g, m + 1);
        buf = buf + 1 == kBuffers ? 0 : buf + 1;
        if (gt == kBuffers - 1) {
          // the sweep wave is that many tiles behind now: time for the zeros around the window
          zero_outside(wave - nsweep, nwaves - nsweep);
          zeroed = true;
        }
      }
      tile_base += g.ntiles;
    }
    // the tiles still in the buffers
    const int first_left = max(tile_base - kBuffers, 0);
    buf = first_left % kBuffers;
    for (int gt = first_left; gt < tile_base; ++gt) {
      if (!wait_for(&cnt.written[w], gt + 1, spin_limit)) {
        give_up();
        return;
      }
      Drained out;
      take_buffer(out, buf);
      store(out);
      buf = buf + 1 == kBuffers ? 0 : buf + 1;
    }
    if (!zeroed) zero_outside(wave - nsweep, nwaves - nsweep);
    if (peek(&cnt.failed)) poison();
    // the loss, if asked for: the scores are the forward kernel's, complete before this
    // kernel started, and this wave has nothing left to do
    if (loss && b == 0 && wave == nsweep) reduce_scores(scores, loss, B, reduction, lane);
    return;
  }

  // -------------------------------- sweep wave ---------------------------------
  const int w = wave;
  const int prev = (w + nsweep - 1) % nsweep;
  R *my_seam = seam + (size_t)w * seam_pitch + kSeamPadLeft;
  const R *up_seam = seam + (size_t)prev * seam_pitch + kSeamPadLeft;
  R *base = tiles + (size_t)w * 2 * kBuffers * kTileElems;
  const R seed = ans_grad ? ans_grad[b] : (R)1;
  int tile_base = 0, buf = 0, rounds = 0;  // tile number modulo kBuffers, and divided by it
  for (int band = 0; band * band_rows <= NS; ++band) {
    const Band g = band_of(band, w, nsweep, NS, NT);
    if (g.row0 > NS) break;
    const int r = g.row0 + lane;
    const bool has_up = g.row0 > 0;
    const int up_base = (w > 0 ? band : band - 1) * cols;
    const int my_base = band * cols;
    // the gradient of the origin cell: lane NS - row0 at step NT + NS - row0
    const int fin_lane = NS - g.row0;
    const int fin_step = (fin_lane < kWave) ? NT + fin_lane : -1;

    // the seed enters as "handed left" into the first cell of the reversed sweep
    R to_below = 0, to_below2 = 0, to_left = (r == 0) ? seed : (R)0;
    R g_origin = 0;
    const R *seam_at = up_seam + (lane - shift);  // seam_at[e]: what lane 0 needs at step e + lane
    const bool has_down = g.row0 + kWave <= NS;  // rows below this wave's: someone reads the seam
    int seen_ready = 0;
    R seen_seam = 0;
    int seen_loaded = 0;
    // one tile; the compile-time flags and the loops are those of the forward kernel
    auto one_tile = [&](int m, auto up_c, auto down_c, auto plain_c) __attribute__((always_inline)) -> bool {
      constexpr bool kUp = decltype(up_c)::value;
      constexpr bool kDown = decltype(down_c)::value;
      constexpr bool kPlain = decltype(plain_c)::value;
      const int gt = tile_base + m;
      if (__builtin_amdgcn_readfirstlane(seen_loaded) < kStagers * (rounds + 1) &&
          !wait_for(&cnt.loaded[w * kBuffers + buf], kStagers * (rounds + 1), spin_limit)) {
        give_up();
        return false;
      }
      R d1q[kTileSteps], d2q[kTileSteps];
      R *gx_row = base + buf * kTileElems + lane * kTilePitch;               // d1 in, gx out
      R *gy_row = base + (kBuffers + buf) * kTileElems + lane * kTilePitch;  // d2 in, gy out
      buf = buf + 1 == kBuffers ? 0 : buf + 1;
      rounds += buf == 0;
      pull_row(d1q, gx_row);
      pull_row(d2q, gy_row);

      bool failed = false;
      auto chunk = [&](int c4, int e0) __attribute__((always_inline)) {
        R handed = 0;
        if (kUp) {
          const int need = kPlain ? e0 + kChunk - shift : min(e0 + kChunk - shift, cols);
          handed = seen_seam;
          if ((kPlain || need > 0) && __builtin_amdgcn_readfirstlane(seen_ready) < up_base + need) {
            // (a wait that has run out is not tried again, see the forward kernel)
            if (!failed && !wait_for(&cnt.ready[prev], up_base + need, spin_limit)) failed = true;
            const int col = e0 + lane - shift;
            handed = (lane < kChunk && col >= 0 && col <= NT) ? up_seam[col] : (R)0;
            lds_reads_done();
          }
          // next chunk's counter, then its seam values (LDS serves a wave in order)
          seen_ready = peek(&cnt.ready[prev]);
          if (kPlain) {
            seen_seam = seam_at[e0 + kChunk];  // every column exists; lanes 8 .. 63 do not matter
          } else {
            const int col = e0 + kChunk + lane - shift;
            seen_seam = 0;
            if (lane < kChunk && col >= 0 && col <= NT) seen_seam = up_seam[col];
          }
          // (the reads above are for the next chunk: they are issued here, before the steps)
          __builtin_amdgcn_sched_barrier(0);
        }
        if (c4 == kTileSteps / kChunk - 1) seen_loaded = peek(&cnt.loaded[w * kBuffers + buf]);
        R down[kChunk], left[kChunk], cell[kChunk];
#pragma unroll
        for (int k = 0; k < kChunk; ++k) {
          const int kk = c4 * kChunk + k;
          R from_above;
          if (kUp) {
            from_above = from_lane_below_or(kModified ? to_below2 : to_below, handed);
            handed = from_lane_above(handed);
          } else {
            from_above = from_lane_below_zero(kModified ? to_below2 : to_below);
          }
          // cells outside the window carry d1 = d2 = 0, so nothing leaks in or out
          cell[k] = from_above + to_left;
          down[k] = d1q[kk] * cell[k];
          left[k] = d2q[kk] * cell[k];
          to_below2 = to_below;
          to_below = down[k];
          to_left = left[k];
          if (k == kChunk / 2 - 1) {
            // the chunk's gradients take the place of its d1 / d2 in the tile: first half
            push_half<0>(gx_row + c4 * kChunk, down);
            push_half<0>(gy_row + c4 * kChunk, left);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
        if (!kPlain) {
          const int kf = fin_step - e0;  // wave-uniform
          if ((unsigned)kf < (unsigned)kChunk) {
#pragma unroll
            for (int k = 0; k < kChunk; ++k)
              if (k == kf) g_origin = cell[k];
          }
        }
        // seam: the last lane's reversed columns e0 - 63 ... (the pads take what falls
        // outside)
        if (kDown && e0 + kChunk > kWave - 1) {
          if (lane == kWave - 1) {
            push_chunk(my_seam + (e0 - (kWave - 1)), down);
            const int done = max(0, min(e0 + kChunk - (kWave - 1), cols));
            publish_lds_writes(&cnt.ready[w], my_base + done);
          }
        }
        push_half<1>(gx_row + c4 * kChunk, down);
        push_half<1>(gy_row + c4 * kChunk, left);
      };
#pragma unroll
      for (int c4 = 0; c4 < kTileSteps / kChunk; ++c4) {
        const int e0 = m * kTileSteps + c4 * kChunk;
        // the window's edges need no care here: d1 = d2 = 0 outside it
        if (kPlain || e0 < g.nsteps) chunk(c4, e0);
      }
      if (failed) {
        give_up();
        return false;
      }
      if (lane == 0) publish_lds_writes(&cnt.written[w], gt + 1);
      return true;
    };
    auto sweep_tiles = [&](auto up_c, auto down_c) __attribute__((always_inline)) -> bool {
      const PlainTiles plain = plain_tiles(g, fin_step, decltype(up_c)::value, shift, NT);
      for (int m = 0; m < plain.lo; ++m)
        if (!one_tile(m, up_c, down_c, std::false_type{})) return false;
      for (int m = plain.lo; m < plain.hi; ++m)
        if (!one_tile(m, up_c, down_c, std::true_type{})) return false;
      for (int m = plain.hi; m < g.ntiles; ++m)
        if (!one_tile(m, up_c, down_c, std::false_type{})) return false;
      return true;
    };
    bool done;
    if (has_up)
      done = has_down ? sweep_tiles(std::true_type{}, std::true_type{})
                      : sweep_tiles(std::true_type{}, std::false_type{});
    else
      done = has_down ? sweep_tiles(std::false_type{}, std::true_type{})
                      : sweep_tiles(std::false_type{}, std::false_type{});
    if (!done) return;
    if (lane == fin_lane && overwrite_ans_grad && ans_grad)
      ans_grad[b] = peek(&cnt.failed) ? std::numeric_limits<R>::quiet_NaN() : g_origin;
    tile_base += g.ntiles;
  }
}

constexpr size_t kLdsBudget = 156 * 1024;

// Sweep waves per workgroup: one per 64 rows, as many as LDS allows.
int pick_sweep_waves(int S, int T, size_t elem, int arrays) {
  int n = (S + 1 + kWave - 1) / kWave;
  n = n < 1 ? 1 : (n > kMaxSweep ? kMaxSweep : n);
  auto bytes = [&](int k) {
    return (size_t)k * ((size_t)((T + 1 + kSeamSlack + 3) & ~3) + (size_t)arrays * 2 * kTileElems) * elem;
  };
  while (n > 1 && bytes(n) > kLdsBudget) --n;
  return n;
}

// Dynamic LDS of a launch: per sweep wave a seam row and 2 x buffers tiles.
size_t lds_bytes(int nsweep, int T, int buffers, size_t elem) {
  return (size_t)nsweep * ((size_t)((T + 1 + kSeamSlack + 3) & ~3) + (size_t)2 * buffers * kTileElems) * elem;
}

template <typename R>
int forward_impl(const R *px, const R *py, const int64_t *boundary, R *p, R *ans, int B, int S,
                 int T, int modified, void *stream, int checks = 0, int *status = nullptr) {
  if (B < 0 || S < 0 || T < 0) return fail(FRNNT_EINVAL, "mi_forward: negative size");
  if (B == 0) return FRNNT_OK;
  if (!px || !py || !p || !ans) return fail(FRNNT_EINVAL, "mi_forward: null pointer");
  if ((size_t)(S + 1) * (T + 1) * sizeof(R) >= ((size_t)1 << 30))
    return fail(FRNNT_ELIMIT, "mi_forward: one utterance's lattice exceeds 1 GiB");
  const int n = pick_sweep_waves(S, T, sizeof(R), 2);
  if (lds_bytes(n, T, 2, sizeof(R)) > kLdsBudget)
    return fail(FRNNT_ELIMIT, "mi_forward: T=%d needs %zu bytes of LDS", T, lds_bytes(n, T, 2, sizeof(R)));
  // With at most two sweep waves there is room, for floats, for a third tile buffer, which
  // gives a staging wave two tiles' time instead of one to empty and refill a buffer.
  constexpr int kFewBuffers = sizeof(R) == 4 ? 3 : 2;
  static_assert(kMaxSweep * 2 <= 16 && 2 * kFewBuffers <= 16, "Counters::loaded is too short");
  const bool few = n <= 2 && lds_bytes(n, T, kFewBuffers, sizeof(R)) <= kLdsBudget;
  // (doubles keep two staging waves per sweep wave: with more waves in the workgroup a sweep
  // wave's two tile rows of doubles no longer fit its share of the registers)
  constexpr int kMany = sizeof(R) == 4 ? kFwdStagers : 2, kFew = sizeof(R) == 4 ? kFwdStagersFew : 2;
  const int stagers = few ? kFew : kMany;
  const size_t lds = lds_bytes(n, T, few ? kFewBuffers : 2, sizeof(R));
  auto kernel = few ? (modified ? mi_forward_kernel<R, true, 2, kFew, kFewBuffers>
                                : mi_forward_kernel<R, false, 2, kFew, kFewBuffers>)
                    : (modified ? mi_forward_kernel<R, true, kMaxSweep, kMany, 2>
                                : mi_forward_kernel<R, false, kMaxSweep, kMany, 2>);
  if (!allow_lds(reinterpret_cast<const void *>(kernel), lds))
    return check_launch("mi_forward: hipFuncSetAttribute");
  hipLaunchKernelGGL(kernel, dim3(B), dim3(n * (1 + stagers) * kWave), lds,
                     static_cast<hipStream_t>(stream), px, py, boundary, p, ans, S, T, g_spin_limit,
                     checks, status);
  return check_launch("mi_forward");
}

template <typename R>
int backward_impl(const R *px, const R *py, const int64_t *boundary, const R *p, R *ans_grad,
                  R *px_grad, R *py_grad, int B, int S, int T, int modified,
                  int overwrite_ans_grad, void *stream, const R *scores = nullptr,
                  R *loss = nullptr, int reduction = 0) {
  (void)py;  // the d2 = 1 - d1 split needs only p and px
  if (loss && (!scores || reduction < 0 || reduction > 2))
    return fail(FRNNT_EINVAL, "mi_backward: loss without scores, or bad reduction");
  if (B < 0 || S < 0 || T < 0) return fail(FRNNT_EINVAL, "mi_backward: negative size");
  if (B == 0) return FRNNT_OK;
  if (!px || !p || !px_grad || !py_grad)
    return fail(FRNNT_EINVAL, "mi_backward: null pointer");
  if ((size_t)(S + 1) * (T + 1) * sizeof(R) >= ((size_t)1 << 30))
    return fail(FRNNT_ELIMIT, "mi_backward: one utterance's lattice exceeds 1 GiB");
  const int n = pick_sweep_waves(S, T, sizeof(R), 2);
  if (lds_bytes(n, T, 2, sizeof(R)) > kLdsBudget)
    return fail(FRNNT_ELIMIT, "mi_backward: T=%d needs %zu bytes of LDS", T, lds_bytes(n, T, 2, sizeof(R)));
  // With at most two sweep waves there is room for more staging waves per sweep wave and,
  // for floats, for a third tile buffer, which gives a staging wave two tiles' time instead
  // of one to empty and refill a buffer.  (A workgroup of 16 waves leaves each 128
  // registers, too few for a sweep wave's two tile rows of doubles.)
  constexpr bool kFloat = sizeof(R) == 4;
  constexpr int kFew = kFloat ? kBwdStagersFew : kBwdStagers;
  constexpr int kFewBuffers = kFloat ? 3 : 2;
  static_assert(kMaxSweep * 2 <= 16 && 2 * kFewBuffers <= 16, "Counters::loaded is too short");
  const bool few = n <= 2 && lds_bytes(n, T, kFewBuffers, sizeof(R)) <= kLdsBudget;
  const int stagers = few ? kFew : kBwdStagers;
  const size_t lds = lds_bytes(n, T, few ? kFewBuffers : 2, sizeof(R));
  auto kernel = few ? (modified ? mi_backward_kernel<R, true, 2, kFew, kFewBuffers>
                                : mi_backward_kernel<R, false, 2, kFew, kFewBuffers>)
                    : (modified ? mi_backward_kernel<R, true, kMaxSweep, kBwdStagers, 2>
                                : mi_backward_kernel<R, false, kMaxSweep, kBwdStagers, 2>);
  if (!allow_lds(reinterpret_cast<const void *>(kernel), lds))
    return check_launch("mi_backward: hipFuncSetAttribute");
  hipLaunchKernelGGL(kernel, dim3(B), dim3(n * (1 + stagers) * kWave), lds,
                     static_cast<hipStream_t>(stream), px, boundary, p, ans_grad, px_grad,
                     py_grad, S, T, overwrite_ans_grad, scores, loss, B, reduction, g_spin_limit);
  return check_launch("mi_backward");
}

}  // namespace

int mi_backward_and_loss(const float *px, const int64_t *boundary, const float *p, float *px_grad,
                         float *py_grad, const float *scores, float *loss, int B, int S, int T,
                         int modified, int reduction, void *stream) {
  return backward_impl<float>(px, nullptr, boundary, p, nullptr, px_grad, py_grad, B, S, T,
                              modified, 0, stream, scores, loss, reduction);
}
int mi_backward_and_loss(const double *px, const int64_t *boundary, const double *p,
                         double *px_grad, double *py_grad, const double *scores, double *loss,
                         int B, int S, int T, int modified, int reduction, void *stream) {
  return backward_impl<double>(px, nullptr, boundary, p, nullptr, px_grad, py_grad, B, S, T,
                               modified, 0, stream, scores, loss, reduction);
}

}  // namespace frnnt

extern "C" {

void frnnt_set_spin_limit(int polls) {
  frnnt::g_spin_limit = polls > 0 ? polls : frnnt::kSpinLimit;
}

int frnnt_mi_forward_f32(const float *px, const float *py, const int64_t *boundary, float *p,
                         float *ans, int B, int S, int T, int modified, void *stream) {
  return frnnt::forward_impl<float>(px, py, boundary, p, ans, B, S, T, modified, stream);
}
int frnnt_mi_forward_f64(const double *px, const double *py, const int64_t *boundary, double *p,
                         double *ans, int B, int S, int T, int modified, void *stream) {
  return frnnt::forward_impl<double>(px, py, boundary, p, ans, B, S, T, modified, stream);
}
int frnnt_mi_forward_checked_f32(const float *px, const float *py, const int64_t *boundary,
                                 float *p, float *ans, int B, int S, int T, int modified,
                                 int checks, int32_t *status, void *stream) {
  return frnnt::forward_impl<float>(px, py, boundary, p, ans, B, S, T, modified, stream, checks,
                                    status);
}
int frnnt_mi_forward_checked_f64(const double *px, const double *py, const int64_t *boundary,
                                 double *p, double *ans, int B, int S, int T, int modified,
                                 int checks, int32_t *status, void *stream) {
  return frnnt::forward_impl<double>(px, py, boundary, p, ans, B, S, T, modified, stream, checks,
                                     status);
}
int frnnt_mi_backward_f32(const float *px, const float *py, const int64_t *boundary,
                          const float *p, float *ans_grad, float *px_grad, float *py_grad, int B,
                          int S, int T, int modified, int overwrite_ans_grad, void *stream) {
  return frnnt::backward_impl<float>(px, py, boundary, p, ans_grad, px_grad, py_grad, B, S, T,
                                     modified, overwrite_ans_grad, stream);
}
int frnnt_mi_backward_f64(const double *px, const double *py, const int64_t *boundary,
                          const double *p, double *ans_grad, double *px_grad, double *py_grad,
                          int B, int S, int T, int modified, int overwrite_ans_grad,
                          void *stream) {
  return frnnt::backward_impl<double>(px, py, boundary, p, ans_grad, px_grad, py_grad, B, S, T,
                                      modified, overwrite_ans_grad, stream);
}

}  // extern "C"
