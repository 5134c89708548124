// The normalizer product of the simple (additive-joiner) loss in float32, with px / py and
// log(P + tiny) written from its accumulators (rnnt_loss.py:66-227; the formulas are at the
// top of simple_logprobs.hip).  A source file of its own because its loop does best with
// the compiler's "max-ilp" scheduling strategy (B = 16, S = 120, T = 400, C = 5000: 120.5 ->
// 115 us; the gradient products in simple_logprobs.hip lose 0.3 - 0.8 us with it), which
// is chosen per file (csrc/Makefile).
#include "common.hip.h"
#include "simple_shared.hip.h"

namespace frnnt {
namespace {

// Normalizer GEMM, wave-private LDS transposition.  Both operands are k-contiguous
// ([rows][C]), the matrix cores want one row per lane.  Letting every lane fetch its
// own row costs one cache-line lookup per lane and instruction, which is what bounds
// that form; here a wave fetches a slab of (kS lattice rows + 32 frames) x kK k with
// coalesced 16-byte loads (kK / 4 lanes per row), applies exp(x - shift) in registers,
// writes the slab to its OWN LDS region (pitch kK + 1, conflict-free for the row-per-lane
// reads that follow) and feeds the matrix cores from there; the next slab is requested
// between the LDS writes and the MFMAs.  The eight waves of a workgroup split k; they
// never wait for each other in the loop (a wave's LDS writes and reads are served in
// program order), only once at the end, when the partial sums meet.
// On this part fp32 MFMA and the VALU work of another wave of the same SIMD do not
// overlap, so the loop's time is the sum of its MFMA cycles and of everything else it
// issues: it is written for instruction count (one load instruction and one add per 16
// bytes, no guards; two 3-input maxima, one fma and one compare per row for the shifts).
// A workgroup covers kS lattice rows (32-row tiles) x 32 frames: 96 or 128 rows, k in
// slabs of 16.  The host picks the form that pads S+1 least, so that at S+1 <= 128 the
// lm operand is fetched once per 32 frames and the am operand once.
constexpr int kPanT = 32;                 // frames per workgroup
constexpr int kPanOutPitch = kPanT + 1;   // pitch of a wave's partial sums in LDS
constexpr int kPanWaves = 8;
constexpr int kPanThreads = kPanWaves * kWave;
template <int kS, int kK>
struct PanelShape {
  static constexpr int kRows = kS + kPanT;        // rows of a slab: lm rows, then am rows
  // Row pitch in LDS: kK + 4.  Rows start 16-byte aligned, so a lane's four values of a row
  // go in as one 16-byte write, and a lane reads its row's eight k of a slab half as two
  // 16-byte reads: eight lanes' reads (rows r .. r + 7, 20 floats apart) fall on all 32 banks.
  static constexpr int kPitch = kK + 4;
  static constexpr int kSlab = kRows * kPitch;    // floats per slab
  static constexpr int kRowLanes = kK / 4;        // lanes that share a row of a slab
  static constexpr int kRowsPerLoad = kWave / kRowLanes;
  static constexpr int kLoads = kRows / kRowsPerLoad;  // 16-byte loads per lane and slab
  static constexpr int kSums = kS * kPanOutPitch; // floats of a wave's partial sums
  static constexpr size_t kLdsBytes =
      (size_t)kPanWaves * (kSlab > kSums ? kSlab : kSums) * sizeof(float);
  static constexpr int kItems = (kS * kPanT / 4 + kPanThreads - 1) / kPanThreads;  // 16-byte outputs per thread
  static_assert(kRows % kRowsPerLoad == 0 && kLoads % 2 == 0 && kS % 32 == 0 && kS <= 128, "shape");
};

template <int kS, int kK>
__global__ void __launch_bounds__(kPanThreads)
    simple_fwd_panel_kernel(const float *__restrict__ lm, const float *__restrict__ am,
                            const int64_t *__restrict__ symbols,
                            const int64_t *__restrict__ boundary,
                            float *__restrict__ lm_max, float *__restrict__ am_max,
                            float *__restrict__ px, float *__restrict__ py,
                            float *__restrict__ norm_raw, const int64_t *__restrict__ window,
                            int B, int S, int T, int C, int term, int rnnt_type, int part_shift) {
  using Shape = PanelShape<kS, kK>;
  constexpr int kPanS = kS, kPanK = kK, kPanRows = Shape::kRows, kPanPitch = Shape::kPitch;
  constexpr int kPanSlab = Shape::kSlab, kPanItems = Shape::kItems;
  constexpr int kRowLanes = Shape::kRowLanes, kRowsPerLoad = Shape::kRowsPerLoad;
  using namespace dgemm;
  extern __shared__ __align__(16) float pan_lds[];
  __shared__ float wave_max[kPanWaves][kPanRows];    // row maxima over each wave's share of k
  __shared__ float wave_shift[kPanWaves][kPanRows];  // the waves' final shifts, as -shift log2(e)
  __shared__ float factor[kPanWaves][kPanRows];      // scale factors for a wave's partial sums
  __shared__ float slab_max[kPanRows];             // row maxima
  __shared__ float row_term[kPanS], row_sym[kPanS], row_max[kPanS];  // lm[s,term], lm[s,sym[s]], lm_max[s]
  __shared__ int row_symbol[kPanS];
  __shared__ float col_term[kPanT], col_max[kPanT];                  // am[t,term], am_max[t]
  const int S1 = S + 1;
  const int t_tiles = T > 0 ? (T + kPanT - 1) / kPanT : 1, s_tiles = (S1 + kPanS - 1) / kPanS;
  int b, s_idx, t_idx;
  if (!place_frames((int)blockIdx.x, t_tiles, s_tiles, part_shift, B, b, s_idx, t_idx)) return;
  const int s_tile = s_idx * kPanS, t_tile = t_idx * kPanT;
  const int T1 = rnnt_type == kRegular ? T + 1 : T;
  // With a window only rows <= s_end and frames <= t_end are looked at afterwards (frame
  // t_end itself only for the -inf that closes the regular lattice): a tile past t_end has
  // nothing to do -- except the tiles of frame 0, which also store the row maxima of lm
  // and the lattice's last column -- and 32-row tiles past s_end are not multiplied.
  // (The window's words are looked at only after the first slab has been requested, so that
  // the two round trips to memory overlap; a tile that turns out to have nothing to do has
  // then requested a slab in vain, range-checked like all the others.)
  const float *lmb = lm + (long)b * S1 * C;
  const float *amb = am + (long)b * T * C;
  const int64_t *symb = symbols + (long)b * S;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5, r32 = lane & 31;
  const float ninf = -__builtin_huge_valf();

  // ---- the symbols come first: the epilogue's gathers depend on them
  // this thread's outputs: 16-byte pieces (row item / 8, frames 4 (item % 8) ..)
  int out_sym[kPanItems];
#pragma unroll
  for (int j = 0; j < kPanItems; ++j) {
    const int item = tid + kPanThreads * j, sr = s_tile + item / 8;
    out_sym[j] = -1;
    if (item < kPanS * 8 && sr < S) {
      const int64_t y = symb[sr];
      out_sym[j] = (y >= 0 && y < C) ? (int)y : -1;
    }
  }
  int my_sym = -1;  // threads 0 .. kS-1 own a lattice row each
  if (tid < kPanS && s_tile + tid < S) {
    const int64_t y = symb[s_tile + tid];
    my_sym = (y >= 0 && y < C) ? (int)y : -1;
  }

  // ---- what this lane fetches of every slab: rows sub + kRowsPerLoad j, k-offset kq
  constexpr int kLoads = Shape::kLoads;
  const int sub = lane / kRowLanes, kq = 4 * (lane % kRowLanes);
  // row j of a fetch is lattice row s_tile + sub + kRowsPerLoad j while that stays below
  // kS, a frame after that.  The loads go through buffer resources that cover lm[b] and
  // am[b]: one instruction each, no branch, any alignment; a row past the last one lies
  // past the resource and reads as 0 -- such rows only feed outputs that are never
  // written.  Columns at and past C (the last slab) belong to the next row and are
  // replaced by -inf, exp(-inf - shift) = 0 in the product.
  constexpr int kLmLoads = kPanS / kRowsPerLoad;
  static_assert(kPanS % kRowsPerLoad == 0, "a fetch row holds lm or am, not both");
  const __amdgpu_buffer_rsrc_t lm_rs =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(lmb), 0, S1 * C * 4, 0x00020000);
  const __amdgpu_buffer_rsrc_t am_rs =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(amb), 0, T * C * 4, 0x00020000);
  const int lm_off = ((s_tile + sub) * C + kq) * 4, am_off = ((t_tile + sub) * C + kq) * 4;  // bytes
  const int step = kRowsPerLoad * C * 4;
  typedef int intx4 __attribute__((ext_vector_type(4)));
  auto fetch = [&](floatx4 (&into)[kLoads], int k0) {
#pragma unroll
    for (int j = 0; j < kLoads; ++j) {
      // (the wave-uniform part of the offset rides in a scalar register)
      const intx4 raw = j < kLmLoads
                            ? __builtin_amdgcn_raw_buffer_load_b128(lm_rs, lm_off, j * step + k0 * 4, 0)
                            : __builtin_amdgcn_raw_buffer_load_b128(
                                  am_rs, am_off, (j - kLmLoads) * step + k0 * 4, 0);
      into[j] = floatx4{__int_as_float(raw[0]), __int_as_float(raw[1]), __int_as_float(raw[2]),
                        __int_as_float(raw[3])};
    }
    if (k0 + kPanK > C) {  // (wave-uniform) the slab that holds column C - 1
#pragma unroll
      for (int j = 0; j < kLoads; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (k0 + kq + i >= C) into[j][i] = ninf;
    }
  };
  const int chunks = (C + kPanK - 1) / kPanK;

  // ---- one pass over k.  The reference subtracts the row maxima before exp
  // (rnnt_loss.py:174-178); a maximum is known only after the whole row has been seen, so
  // each wave works with a SHIFT per row instead: the largest value of the row it had
  // seen when the shift was last set.  A value more than kMargin above the shift (always
  // the case for the first finite value of a row) makes the wave raise its shifts and
  // scale its partial sums to match; anything closer stays representable, e^(2 kMargin)
  // per product.  The running maxima are kept beside the shifts, and when the waves
  // meet their partial sums are brought to the true maxima, exp(shift - max) <= 1.
  constexpr float kMargin = 30.f;
  // (One slab in flight per wave is enough: with a second one the 96-row form was 1 us
  // slower at B = 32, S = 80, T = 250, C = 500 -- the loop is bound by what it issues, not
  // by the round trips.)
  floatx4 slab[kLoads];
  if (wave < chunks) fetch(slab, wave * kPanK);
  const Limits lim = limits_of(window, b, S, T);
  if (t_tile > lim.t_end && t_tile > 0) return;

  // ---- epilogue inputs, requested behind the first slab (the symbols they depend on
  // were requested before it) so that their latency hides under the loop:
  // am[b, t, sym[b, s]] for this thread's outputs ...
  float am_sym[kPanItems][4];
#pragma unroll
  for (int j = 0; j < kPanItems; ++j) {
    const int item = tid + kPanThreads * j;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int tr = t_tile + 4 * (item % 8) + i;
      am_sym[j][i] = (out_sym[j] >= 0 && tr < T) ? amb[tr * C + out_sym[j]] : 0.f;
    }
  }
  // ... and the per-row / per-column terms (kept in registers until the loop is done)
  float my_term = 0.f, my_symval = 0.f;
  if (tid < kPanS) {
    const int sr = s_tile + tid;
    if (sr < S1) {
      my_term = lmb[sr * C + term];
      if (my_sym >= 0) my_symval = lmb[sr * C + my_sym];
    }
  } else if (tid >= 128 && tid < 128 + kPanT) {
    const int tr = t_tile + tid - 128;
    my_term = tr < T ? amb[tr * C + term] : 0.f;
  }

  float seen[kLoads];     // largest value this lane has met in the row
  // -shift * log2(e), see exp_shifted; the lanes of a row agree on it.  kUnset while the
  // row has shown nothing finite: it sends -inf to exp2(-inf) = 0 and anything finite
  // above the margin.
  float shift2[kLoads];
  constexpr float kUnset = 3.0e38f;
#pragma unroll
  for (int j = 0; j < kLoads; ++j) seen[j] = ninf, shift2[j] = kUnset;
  const int live_tiles = min(kPanS / 32, (min(S1, lim.s_end + 1) - s_tile + 31) / 32);
  float *mine = pan_lds + wave * kPanSlab;
  floatx16 acc[kPanS / 32];
#pragma unroll
  for (int j = 0; j < kPanS / 32; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;

  auto across_row = [&](float v) {  // maximum over the lanes that share a row
#pragma unroll
    for (int off = 1; off < kRowLanes; off <<= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
  };
  // (sums_are_zero: the wave's first slab, which always comes here -- nothing to scale yet)
  auto raise_shifts = [&](bool sums_are_zero) {
    if (sums_are_zero) {
#pragma unroll
      for (int j = 0; j < kLoads; ++j)
        shift2[j] = fminf(shift2[j], -across_row(seen[j]) * kLog2e);
      return;
    }
#pragma unroll
    for (int j = 0; j < kLoads; ++j) {
      const float now = fminf(shift2[j], -across_row(seen[j]) * kLog2e);
      const float f = __builtin_amdgcn_exp2f(now - shift2[j]);  // exp(old shift - new shift)
      shift2[j] = now;
      if (lane % kRowLanes == 0) factor[wave][sub + kRowsPerLoad * j] = f;
    }
    __builtin_amdgcn_wave_barrier();
    const float ft = factor[wave][kPanS + r32];
#pragma unroll
    for (int j = 0; j < kPanS / 32; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v)
        acc[j][v] *= factor[wave][32 * j + 8 * (v / 4) + 4 * half + (v % 4)] * ft;
    __builtin_amdgcn_wave_barrier();
  };
  // one slab: exp(x - shift) to LDS, the request for the slab that will take these
  // registers next, then the products (32-row tiles without lattice rows are skipped)
  auto consume = [&](floatx4 (&slab)[kLoads], int next_chunk, bool first) {
    bool above = false;
#pragma unroll
    for (int j = 0; j < kLoads; ++j) {
      // two three-input maxima; a row is above its margin exactly when its maximum is
      seen[j] = max3_raw(max3_raw(slab[j][0], slab[j][1], slab[j][2]), slab[j][3], seen[j]);
      above |= __builtin_fmaf(seen[j], kLog2e, shift2[j]) > kMargin * kLog2e;
    }
    if (__any(above)) raise_shifts(first);
#pragma unroll
    for (int j = 0; j < kLoads; ++j) {
      floatx4 e;
#pragma unroll
      for (int i = 0; i < 4; ++i) e[i] = exp_shifted(slab[j][i], shift2[j]);
      *reinterpret_cast<floatx4 *>(mine + (sub + kRowsPerLoad * j) * kPanPitch + kq) = e;
    }
    if (next_chunk < chunks) fetch(slab, next_chunk * kPanK);
    // MFMA i of the slab multiplies k = i (lanes 0..31) and k = i + kK / 2 (lanes 32..63): the
    // order in which a slab's k are summed is free, and this one lets a lane take its row's
    // share of the slab with 16-byte reads
    static_assert(kPanK == 16, "two 16-byte reads per row and slab half");
    const float *ap = mine + r32 * kPanPitch + 8 * half;
    const float *bp = mine + (kPanS + r32) * kPanPitch + 8 * half;
    const floatx4 b0 = *reinterpret_cast<const floatx4 *>(bp);
    const floatx4 b1 = *reinterpret_cast<const floatx4 *>(bp + 4);
#pragma unroll
    for (int j = 0; j < kPanS / 32; ++j)
      if (j < live_tiles) {
        const floatx4 a0 = *reinterpret_cast<const floatx4 *>(ap + j * 32 * kPanPitch);
        const floatx4 a1 = *reinterpret_cast<const floatx4 *>(ap + j * 32 * kPanPitch + 4);
#pragma unroll
        for (int i = 0; i < 4; ++i)
          acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0[i], b0[i], acc[j], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i)
          acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[i], b1[i], acc[j], 0, 0, 0);
      }
  };
  for (int chunk = wave; chunk < chunks; chunk += kPanWaves)
    consume(slab, chunk + kPanWaves, chunk == wave);

  // ---- the waves meet: maxima first ...
#pragma unroll
  for (int j = 0; j < kLoads; ++j) {
    const float top = across_row(seen[j]);
    if (lane % kRowLanes == 0) {
      wave_max[wave][sub + kRowsPerLoad * j] = top;
      wave_shift[wave][sub + kRowsPerLoad * j] = shift2[j];
    }
  }
  __syncthreads();
  if (tid < kPanRows) {
    float r = wave_max[0][tid];
#pragma unroll
    for (int w = 1; w < kPanWaves; ++w) r = fmaxf(r, wave_max[w][tid]);
    // saved for the backward pass; rows that do not exist get a harmless shift
    bool exists;
    if (tid < kPanS) {
      exists = s_tile + tid < S1;
      if (exists && t_tile == 0) lm_max[(long)b * S1 + s_tile + tid] = r;
    } else {
      exists = t_tile + tid - kPanS < T;
      if (exists && s_tile == 0) am_max[(long)b * T + t_tile + tid - kPanS] = r;
    }
    slab_max[tid] = exists ? r : 0.f;
    // what brings a wave's partial sums from its shift to the maximum (a wave that met
    // nothing finite in the row holds zeros there)
#pragma unroll
    for (int w = 0; w < kPanWaves; ++w)
      factor[w][tid] = exists ? __builtin_amdgcn_exp2f(-__builtin_fmaf(r, kLog2e, wave_shift[w][tid])) : 1.f;
  }
  __syncthreads();
  // ... then the partial sums: [wave][kS][33] in the slab space
  if (tid < kPanS) {
    row_term[tid] = my_term;
    row_sym[tid] = my_symval;
    row_max[tid] = slab_max[tid];
    row_symbol[tid] = my_sym;
  } else if (tid >= 128 && tid < 128 + kPanT) {
    col_term[tid - 128] = my_term;
    col_max[tid - 128] = slab_max[kPanS + tid - 128];
  }
  float *part = pan_lds + wave * Shape::kSums;
  {
    const float ft = factor[wave][kPanS + r32];
#pragma unroll
    for (int j = 0; j < kPanS / 32; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = 32 * j + 8 * (v / 4) + 4 * half + (v % 4);
        part[m * kPanOutPitch + r32] = acc[j][v] * (factor[wave][m] * ft);
      }
  }
  __syncthreads();

  const int t_mask = (rnnt_type == kRegular && boundary) ? (int)boundary[4 * b + 3] : -1;
  float *pxb = px + (long)b * S * T1;
  float *pyb = py + (long)b * S1 * T;
  float *nrb = norm_raw ? norm_raw + (long)b * S1 * T : nullptr;
#pragma unroll
  for (int j = 0; j < kPanItems; ++j) {
    const int item = tid + kPanThreads * j;
    const int m = item / 8, out_t = 4 * (item % 8), sr = s_tile + m;
    if (item >= kPanS * 8 || sr >= S1) continue;
    float raw[4], yv[4], xv[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float sum = 0.f;
#pragma unroll
      for (int w = 0; w < kPanWaves; ++w)
        sum += pan_lds[w * Shape::kSums + m * kPanOutPitch + out_t + i];
      raw[i] = logf(sum + 1.17549435e-38f);
      const float norm = raw[i] + row_max[m] + col_max[out_t + i];
      yv[i] = (col_term[out_t + i] + row_term[m]) - norm;
      float v = std::numeric_limits<float>::quiet_NaN();  // out-of-vocabulary symbol
      if (row_symbol[m] >= 0) v = (am_sym[j][i] + row_sym[m]) - norm;
      if (t_tile + out_t + i == t_mask) v = ninf;
      xv[i] = v;
    }
    const int tr = t_tile + out_t;
    if (tr + 4 <= T) {
      if (nrb) *reinterpret_cast<floatx4u *>(nrb + sr * T + tr) = floatx4u{raw[0], raw[1], raw[2], raw[3]};
      *reinterpret_cast<floatx4u *>(pyb + sr * T + tr) = floatx4u{yv[0], yv[1], yv[2], yv[3]};
      if (sr < S)
        *reinterpret_cast<floatx4u *>(pxb + sr * T1 + tr) = floatx4u{xv[0], xv[1], xv[2], xv[3]};
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (tr + i >= T) continue;
        if (nrb) nrb[sr * T + tr + i] = raw[i];
        pyb[sr * T + tr + i] = yv[i];
        if (sr < S) pxb[sr * T1 + tr + i] = xv[i];
      }
    }
  }
  // the extra column of the regular lattice: nothing can be emitted after the last frame
  if (rnnt_type == kRegular && t_tile == 0 && tid < kPanS && s_tile + tid < S)
    pxb[(s_tile + tid) * T1 + T] = ninf;
}

template <int kS, int kK>
void launch_fwd_panel(const float *lm, const float *am, const int64_t *symbols,
                      const int64_t *boundary, float *lm_max, float *am_max, float *px,
                      float *py, float *norm_raw, const int64_t *window, int B, int S, int T,
                      int C, int term, int rnnt_type, hipStream_t stream) {
  using Shape = PanelShape<kS, kK>;
  const int t_tiles = T > 0 ? (T + kPanT - 1) / kPanT : 1;
  const int s_tiles = (S + 1 + kS - 1) / kS;
  auto kernel = simple_fwd_panel_kernel<kS, kK>;
  (void)allow_lds(reinterpret_cast<const void *>(kernel), Shape::kLdsBytes);
  const int shift = frame_part_shift_for(B, t_tiles);
  const int t_per = (t_tiles + (1 << shift) - 1) >> shift;
  const long units = (long)B << shift;
  const unsigned grid =
      (unsigned)(dgemm::kXcds * ((units + dgemm::kXcds - 1) / dgemm::kXcds) * t_per * s_tiles);
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(kPanThreads), Shape::kLdsBytes, stream, lm, am,
                     symbols, boundary, lm_max, am_max, px, py, norm_raw, window, B, S, T, C, term,
                     rnnt_type, shift);
}
}  // namespace

void launch_normalizer_f32(const float *lm, const float *am, const int64_t *symbols,
                           const int64_t *boundary, float *lm_max, float *am_max, float *px,
                           float *py, float *norm_raw, const int64_t *window, int B, int S, int T,
                           int C, int term, int rnnt_type, hipStream_t stream) {
  // the row count per workgroup that leaves fewer padding rows; 128 on a tie
  const int S1 = S + 1;
  const int padded96 = (S1 + 95) / 96 * 96, padded128 = (S1 + 127) / 128 * 128;
  if (padded96 < padded128)
    launch_fwd_panel<96, 16>(lm, am, symbols, boundary, lm_max, am_max, px, py, norm_raw, window,
                             B, S, T, C, term, rnnt_type, stream);
  else
    launch_fwd_panel<128, 16>(lm, am, symbols, boundary, lm_max, am_max, px, py, norm_raw, window,
                              B, S, T, C, term, rnnt_type, stream);
}
}  // namespace frnnt
