// Weight gradient of 3x3 convolutions (stride 1 or 2) with an LDS input tile shared by all nine taps.
//
//   dW[k][c][r][s] = sum_{n,p,q} dy[n][k][p][q] * x[n][c][p*stride - ph + r][q*stride - pw + s]
//
// A workgroup owns BM output channels x BC input channels x 9 taps and walks "units" of the
// reduction: RU consecutive output rows of one image (<= 64 pixels).  Per unit it stages in LDS
//   dyS[pixel][m]            the BM x (RU*Q) slice of dy (MFMA A operand, k = pixel),
//   xS[c][row][col]          the BC x ((RU-1)*stride+3) x (W+2) input slab, zero padding materialised,
// and every tap (r, s) reads its B operand from the SAME slab at offset r*pitch + s from the
// pixel's window origin.  Each input element is therefore fetched once per unit instead of once
// per tap, the address arithmetic of an im2col gather disappears from the inner loop, and one
// operand fetch feeds nine MFMAs.
// The four wavefronts tile (BM/32) x (BC/32); each holds 9 accumulator tiles of 32x32
// (v_mfma_f32_32x32x2_f32: 144 accumulator registers).  The next unit's global loads are spread
// over the k-steps of the current unit and land in the other LDS buffer.
//
// The reduction is split over workgroups (grid.z); partials are written as [split][tap][K][C] and
// summed in ascending split order by k_wgrad3x3_reduce: results are run-to-run identical.
#include <stdlib.h>

#include "common.h"

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef __amdgpu_buffer_rsrc_t rsrc_t;

constexpr int NT = 512;
constexpr int UPIXP = 64;        // padded pixels per unit (k dimension of one unit)
constexpr int kOOB = int(0x80000000u);
constexpr int kFar = 0x40000000;  // byte offset past any image (images are < 1 GiB); kFar + kFar = kOOB
constexpr int TABN = 72;          // window-offset table entries: 64 pixels + the look-ahead of the last k-steps

__device__ __forceinline__ rsrc_t make_rsrc(const void *p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, bytes, 0x00020000);
}
struct W3Args {
  const float *dy, *x;
  float *part;           // [splits][9][K][C]
  int N, C, H, W, K, P, Q, ph, pw, stride;
  int RU;                // output rows per unit
  int units_per_image;   // ceil(P / RU)
  int total_units, units_per_split;
  // 1-D grid of gx * gy * gz workgroups: k tile fastest, then channel tile, then split.  xcd: the j-th
  // workgroup of XCD x (workgroup w runs on XCD w % 8) takes the logical id x * (count / 8) + j, so that the
  // tiles of one split -- they read the same pixels of dy and x -- share that XCD's L2.  Only which hardware
  // computes which partial changes.
  int gx, gy, gz, xcd;
};

// LOGP: log2 of the LDS row pitch (>= W + 2 * pad_w); ROWS = RU + 2 slab rows.
// 512 threads = 8 wavefronts: wavefronts 0-3 and 4-7 each tile the same (BM/32) x (BC/32) output
// block but take the first / second half of every unit's k-steps; their accumulators are summed
// through LDS at the end.  Two wavefronts per SIMD share one LDS tile, so one wavefront's address
// arithmetic and memory waits overlap the other's MFMAs (within a single wavefront VALU work does
// not overlap its own MFMAs).
//
// Vector-ALU work per MFMA is kept minimal, because it is paid in MFMA issue slots:
//   * every staging slot of a thread is "thread constant + unit-uniform term": the thread part is
//     computed once per kernel, the uniform part on the scalar unit, and the k-step loop is fully
//     unrolled so that slot indices and LDS write offsets are immediates (one v_add per load);
//   * image, channel and row bounds are enforced by the buffer descriptor (one per image) and by
//     an out-of-range offset, not by per-lane predicates;
//   * the LDS offset of a pixel's 3x3 window comes from a 64-entry table built once per kernel
//     (one for full units, one for the short last unit of an image).
template <int BM, int BC, int LOGP, int ROWS>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(2, 2))) void k_wgrad3x3(W3Args a) {
  constexpr int PITCHP = 1 << LOGP;
  constexpr int PA = BM + 1;                         // dyS pitch: odd, so the pixel-major staging writes spread over banks
  constexpr int CHS = ROWS * PITCHP + 1;             // xS channel stride: odd -> lanes (channels) hit distinct banks
  constexpr int XBUF = BC * CHS;                     // one x buffer
  constexpr int ZPAD = 3 * PITCHP;                   // always-zero area read by the padded pixels of a short unit
  constexpr int WGC = BC / 32, WGM = 4 / WGC;
  static_assert(BM == WGM * 32, "four wavefronts of 32 rows x 32 channels per half");
  constexpr int CPB = NT >> LOGP;                    // channels staged per pass of the 512 threads
  static_assert(BC % CPB == 0, "channel tile is a whole number of staging passes");
  constexpr int DSLOTS = BM * UPIXP / NT;            // dy elements per thread per unit
  constexpr int XSLOTS = (BC / CPB) * ROWS;          // x elements per thread per unit
  constexpr int NSMAX = UPIXP / 4;                   // k-steps of one wavefront in a full unit
  constexpr int NSFIT = 12;                          // the slots are spread over this many k-steps
  constexpr int DPS = (DSLOTS + NSFIT - 1) / NSFIT;
  constexpr int XPS = (XSLOTS + NSFIT - 1) / NSFIT;
  constexpr int LAT = 3;                             // a load issued in k-step i is written to LDS after k-step i + LAT

  extern __shared__ float smem[];
  float *dyS = smem;                                  // [2][UPIXP][PA]
  float *xS = smem + 2 * UPIXP * PA;                  // [2][BC][CHS]
  float *zeroS = xS + 2 * XBUF;                       // ZPAD zeros
  int *tab = reinterpret_cast<int *>(zeroS + ZPAD);   // [2][TABN] window offsets per pixel

  const int t = threadIdx.x, lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int half = wave >> 2, w4 = wave & 3;
  const int wm = w4 / WGC, wc = w4 % WGC;
  int bx, by, bz;
  {
    const int w = int(blockIdx.x), count = a.gx * a.gy * a.gz;
    const int lw = a.xcd && (count & 7) == 0 ? (w & 7) * (count >> 3) + (w >> 3) : w;
    bz = lw / (a.gx * a.gy);
    const int rem = lw - bz * (a.gx * a.gy);
    by = rem / a.gx;
    bx = rem - by * a.gx;
  }
  const int k0 = bx * BM, c0 = by * BC;
  const int u_begin = bz * a.units_per_split;
  const int u_end = min(u_begin + a.units_per_split, a.total_units);
  const int PQ = a.P * a.Q, HW = a.H * a.W;
  const unsigned dy_img_bytes = unsigned(a.K) * PQ * 4u, x_img_bytes = unsigned(a.C) * HW * 4u;

  // the zero area and the pad columns are written once; staging only rewrites the image columns
  for (int i = t; i < 2 * XBUF + ZPAD; i += NT) xS[i] = 0.f;
  // window offset of pixel `pix` in a full unit (table 0) and in an image's last unit (table 1)
  if (t < 2 * TABN) {
    const int which = t >= TABN, pix = t - which * TABN;
    const int tail_rows = a.P % a.RU;
    const int upix = (which && tail_rows ? tail_rows : a.RU) * a.Q;
    const int row = pix / a.Q, q = pix - row * a.Q;
    tab[t] = pix < upix ? (row * PITCHP + q) * a.stride : 0x7fffffff;
  }

  v16f acc[9];
#pragma unroll
  for (int i = 0; i < 9; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;

  // ---- staging roles of this thread (unit independent) ---------------------------------------
  // dy: pixel t % 64 of output channel k0 + t / 64 + 8 * e           -> dyS[pixel][channel]
  // x : column t % PITCHP of channel c0 + t / PITCHP + CPB * (e / ROWS), slab row e % ROWS
  const int pixt = t & (UPIXP - 1), tm = t >> 6;
  const int td4 = (tm * PQ + pixt) * 4;
  const int dw_off = pixt * PA + tm;
  const int tcol = t & (PITCHP - 1), tch = t >> LOGP;
  const int wcol = tcol - a.pw;
  // a pad column loads out of range (zero) and rewrites its own zero
  const int tx4 = unsigned(wcol) < unsigned(a.W) ? (tch * HW + wcol) * 4 : kFar;
  const int xw_off = tch * CHS + tcol;

  auto unit_geom = [&](int u, int &n, int &p0, int &rows) {
    n = u / a.units_per_image;
    p0 = (u - n * a.units_per_image) * a.RU;
    rows = min(a.RU, a.P - p0);
  };
  // byte offsets inside image n; `vd` is the thread part, already out of range for a padded pixel
  auto dy_voff = [&](int e, int vd, int p0) -> int { return vd + ((k0 + 8 * e) * PQ + p0 * a.Q) * 4; };
  auto x_voff = [&](int e, int p0) -> int {
    const int ce = e / ROWS, row = e - ce * ROWS;
    const int h = p0 * a.stride - a.ph + row;
    const int sx = unsigned(h) < unsigned(a.H) ? ((c0 + CPB * ce) * HW + h * a.W) * 4 : kFar;
    return tx4 + sx;  // kFar + kFar = 2^31, kFar + valid < 2^31 but past any image: both out of range
  };
  auto x_dst = [&](int e) -> int {
    const int ce = e / ROWS, row = e - ce * ROWS;
    return xw_off + ce * (CPB * CHS) + row * PITCHP;
  };
  auto ld = [&](rsrc_t r, int voff) -> float {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, 0, 0));
  };

  if (u_begin < u_end) {
    int n, p0, rows;
    unit_geom(u_begin, n, p0, rows);
    const rsrc_t rdy = make_rsrc(a.dy + size_t(n) * a.K * PQ, dy_img_bytes);
    const rsrc_t rx = make_rsrc(a.x + size_t(n) * a.C * HW, x_img_bytes);
    const int vd = pixt < rows * a.Q ? td4 : kOOB;
    __syncthreads();  // zero fill done before the first slab lands
#pragma unroll
    for (int e = 0; e < DSLOTS; ++e) dyS[dw_off + 8 * e] = ld(rdy, dy_voff(e, vd, p0));
#pragma unroll
    for (int e = 0; e < XSLOTS; ++e) xS[x_dst(e)] = ld(rx, x_voff(e, p0));
  }
  __syncthreads();

  int cur = 0;
  for (int u = u_begin; u < u_end; ++u) {
    int n, p0, rows;
    unit_geom(u, n, p0, rows);
    const int upix = rows * a.Q;
    int nn, np0, nrows;
    const bool more = u + 1 < u_end;
    unit_geom(more ? u + 1 : u, nn, np0, nrows);
    // no next unit: an empty descriptor makes every staging load return zero
    const rsrc_t rdy = make_rsrc(a.dy + size_t(nn) * a.K * PQ, more ? dy_img_bytes : 0u);
    const rsrc_t rx = make_rsrc(a.x + size_t(nn) * a.C * HW, more ? x_img_bytes : 0u);
    const int vd = pixt < nrows * a.Q ? td4 : kOOB;

    const float *dcur = dyS + cur * (UPIXP * PA);
    const float *xcur = xS + cur * XBUF;
    float *dnxt = dyS + (cur ^ 1) * (UPIXP * PA);
    float *xnxt = xS + (cur ^ 1) * XBUF;

    // this wavefront's share of the unit's k-steps (two pixels each)
    const int ksteps = (upix + 1) >> 1;
    const int khalf = (ksteps + 1) >> 1;
    const int s_begin = half ? khalf : 0;
    const int nsteps = half ? ksteps - khalf : khalf;

    // A operand: dyS[pix][m]; B operand: xS[c][window(pix) + r*PITCHP + s]; pix = 2*step + lane/32
    const float *ap = dcur + (2 * s_begin + (lane >> 5)) * PA + wm * 32 + (lane & 31);
    const float *bp = xcur + (wc * 32 + (lane & 31)) * CHS;
    const int zoff = int(zeroS - bp);  // this lane's offset of the zero area (beyond every window offset)
    const int *tb = tab + (rows != a.RU ? TABN : 0) + 2 * s_begin + (lane >> 5);

    // Operand fragments of k-step i+1 are fetched while the MFMAs of k-step i run; the window
    // offset of k-step i+2 is fetched one step earlier still.
    float av[2], bv[2][9];
    int tv[3];
    auto frag = [&](int i, int buf, int tval) {
      av[buf] = ap[2 * i * PA];
      // a pixel past the unit's end has a zero dy column; its x operand comes from the zero area
      // so that no stale LDS value can meet it
      const float *w = bp + min(tval, zoff);
#pragma unroll
      for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int s = 0; s < 3; ++s) bv[buf][r * 3 + s] = w[r * PITCHP + s];
    };
    auto mfmas = [&](int buf) {
#pragma unroll
      for (int i = 0; i < 9; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[buf], bv[buf][i], acc[i], 0, 0, 0);
    };

    tv[0] = tb[0];
    tv[1] = tb[2];
    frag(0, 0, tv[0]);
    float st[LAT + 1][DPS + XPS];
#pragma unroll
    for (int i = 0; i < NSMAX + LAT; ++i) {
      if (i < NSMAX && i < nsteps) {
#pragma unroll
        for (int j = 0; j < DPS; ++j)
          if (i * DPS + j < DSLOTS) st[i % (LAT + 1)][j] = ld(rdy, dy_voff(i * DPS + j, vd, np0));
#pragma unroll
        for (int j = 0; j < XPS; ++j)
          if (i * XPS + j < XSLOTS) st[i % (LAT + 1)][DPS + j] = ld(rx, x_voff(i * XPS + j, np0));
        tv[(i + 2) % 3] = tb[2 * (i + 2)];
        frag(i + 1, (i + 1) & 1, tv[(i + 1) % 3]);
        mfmas(i & 1);
      }
      if (i >= LAT && i - LAT < nsteps) {
        const int w = i - LAT;
#pragma unroll
        for (int j = 0; j < DPS; ++j)
          if (w * DPS + j < DSLOTS) dnxt[dw_off + 8 * (w * DPS + j)] = st[w % (LAT + 1)][j];
#pragma unroll
        for (int j = 0; j < XPS; ++j)
          if (w * XPS + j < XSLOTS) xnxt[x_dst(w * XPS + j)] = st[w % (LAT + 1)][DPS + j];
      }
    }
    // slots not reached by a short unit's k-steps
    if (more) {
      for (int e = nsteps * DPS; e < DSLOTS; ++e) dnxt[dw_off + 8 * e] = ld(rdy, dy_voff(e, vd, np0));
      for (int e = nsteps * XPS; e < XSLOTS; ++e) xnxt[x_dst(e)] = ld(rx, x_voff(e, np0));
    }
    __syncthreads();
    cur ^= 1;
  }

  // The two halves' accumulators are summed through LDS (the staging buffers are free now):
  // the first half ends up owning taps 0-4 and the second taps 5-8, so that one partial per
  // workgroup goes to memory and both halves share the stores.
  {
    constexpr int T0 = 5;  // taps kept by the first half
    float *xch = smem + lane;
    const int wbase = w4 * 16 * 64;
    if (half == 1) {
#pragma unroll
      for (int i = 0; i < T0; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) xch[(i * 4 * 16 + v) * 64 + wbase] = acc[i][v];
    }
    __syncthreads();
    if (half == 0) {
#pragma unroll
      for (int i = 0; i < T0; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][v] += xch[(i * 4 * 16 + v) * 64 + wbase];
    }
    __syncthreads();
    if (half == 0) {
#pragma unroll
      for (int i = T0; i < 9; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) xch[((i - T0) * 4 * 16 + v) * 64 + wbase] = acc[i][v];
    }
    __syncthreads();
    if (half == 1) {
#pragma unroll
      for (int i = T0; i < 9; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][v] += xch[((i - T0) * 4 * 16 + v) * 64 + wbase];
    }
    // partial[z][tap][k][c]
    float *pz = a.part + size_t(bz) * 9 * a.K * a.C;
    const int c = c0 + wc * 32 + (lane & 31);
#pragma unroll
    for (int i = 0; i < 9; ++i) {
      if ((i < T0) != (half == 0)) continue;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = k0 + wm * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        if (m < a.K && c < a.C) pz[(size_t(i) * a.K + m) * a.C + c] = acc[i][v];
      }
    }
  }
}

// dW[k][c][tap] = sum over splits of partial[z][tap][k][c], in a fixed order.
// A workgroup takes EP consecutive (k, c) pairs.  Its 256 threads form ZL = 256 / EP z-lanes x EP
// pairs: lane zl sums the splits z = zl, zl + ZL, ... (ascending) of all nine taps, the lane sums
// are added in lane order, and the 9 * EP results are transposed through LDS so that they leave as
// one contiguous run.  EP is chosen from the layer shape alone, so the summation order depends
// only on the shape: results are run-to-run identical.
template <int EP>
__global__ __launch_bounds__(256) void k_wgrad3x3_reduce(const float *__restrict__ part, float *__restrict__ dW, int K,
                                                        int C, int splits) {
  constexpr int ZL = 256 / EP;
  __shared__ float lanes[ZL][9][EP];
  __shared__ float tile[EP * 9];
  const long KC = long(K) * C;
  const long kc0 = long(blockIdx.x) * EP;
  const int e = threadIdx.x % EP, zl = threadIdx.x / EP;
  const long kc = kc0 + e;
  float s[9];
#pragma unroll
  for (int tap = 0; tap < 9; ++tap) s[tap] = 0.f;
  if (kc < KC) {
    for (int z = zl; z < splits; z += ZL) {
      const float *pz = part + long(z) * 9 * KC + kc;
#pragma unroll
      for (int tap = 0; tap < 9; ++tap) s[tap] += pz[tap * KC];
    }
  }
#pragma unroll
  for (int tap = 0; tap < 9; ++tap) lanes[zl][tap][e] = s[tap];
  __syncthreads();
  for (int i = threadIdx.x; i < EP * 9; i += 256) {
    const int tap = i / EP, ee = i % EP;
    float r = lanes[0][tap][ee];
#pragma unroll
    for (int l = 1; l < ZL; ++l) r += lanes[l][tap][ee];
    tile[ee * 9 + tap] = r;
  }
  __syncthreads();
  const long nvalid = (KC - kc0 < EP ? KC - kc0 : EP) * 9;
  for (int i = threadIdx.x; i < nvalid; i += 256) dW[kc0 * 9 + i] = tile[i];
}

struct W3Plan {
  bool ok;
  int bm, bc, logp, rows, ru, splits, units_per_split, total_units, upi;
  size_t lds;
};

inline W3Plan plan(const sgh_conv_geom *g) {
  W3Plan p{};
  p.ok = false;
  if (g->R != 3 || g->S != 3 || g->stride_h != g->stride_w || (g->stride_h != 1 && g->stride_h != 2)) return p;
  const int st = g->stride_h;
  if (g->pad_h > 2 || g->pad_w > 2) return p;
  if (g->W + 2 > 64 || g->Q < 2 || g->Q > 64 || g->C < 32 || g->K < 64) return p;
  if (sgh_env().wgrad3x3_off) return p;
  // instantiated slabs, stride 1: pitch 64 x 3 rows (RU 1), pitch 32 x 4 rows (RU 2), pitch 16 x 6 rows
  // (RU 4), pitch 16 x 9 rows (RU 7: a whole 7x7 plane); stride 2: pitch 64 x 5 rows (RU 2), pitch 32 x 9
  // rows (RU 4), pitch 16 x 15 rows (RU 7)
  const int cols = g->W + 2 * g->pad_w;  // slab columns a window can touch
  if (cols > 64) return p;
  p.logp = cols <= 16 ? 4 : (cols <= 32 ? 5 : 6);
  if (st == 1) {
    if (p.logp == 6) p.ru = 1;
    else if (p.logp == 5) p.ru = 2;
    else p.ru = (7 * g->Q <= UPIXP && g->P >= 7) ? 7 : 4;
  } else {
    p.ru = p.logp == 6 ? 2 : (p.logp == 5 ? 4 : 7);
    if (g->K < 128) return p;  // only the 128 x 32 tile is instantiated for the taller stride-2 slabs
  }
  if (p.ru > g->P || p.ru * g->Q > UPIXP) return p;
  p.rows = (p.ru - 1) * st + 3;
  p.bm = g->K >= 128 ? 128 : 64;
  p.bc = p.bm == 128 ? 32 : 64;
  if (p.bc == 64 && g->C < 64) return p;
  p.upi = (g->P + p.ru - 1) / p.ru;
  p.total_units = g->N * p.upi;
  const long tiles = long((g->K + p.bm - 1) / p.bm) * ((g->C + p.bc - 1) / p.bc);
  // the LDS footprint allows one workgroup per CU: aim at one full wave of workgroups
  long want = (long(sgh_num_cus()) + tiles - 1) / tiles;
  long max_splits = p.total_units / 2;
  if (max_splits < 1) max_splits = 1;
  long s = want < max_splits ? want : max_splits;
  if (s < 1) s = 1;
  p.units_per_split = int((p.total_units + s - 1) / s);
  p.splits = (p.total_units + p.units_per_split - 1) / p.units_per_split;
  const int pitchp = 1 << p.logp, chs = p.rows * pitchp + 1;
  p.lds = (size_t(2) * UPIXP * (p.bm + 1) + size_t(2) * p.bc * chs + 3 * pitchp + 2 * TABN) * sizeof(float);
  if (p.lds > 160 * 1024 || p.lds < size_t(5) * 4096 * sizeof(float)) return p;  // (the epilogue exchanges 5 taps through LDS)
  // staging offsets are 32-bit byte offsets inside one image, with kFar as the out-of-range mark
  if (size_t(g->K) * g->P * g->Q * 4 >= size_t(kFar) || size_t(g->C) * g->H * g->W * 4 >= size_t(kFar)) return p;
  p.ok = true;
  return p;
}

template <int BM, int BC, int LOGP, int ROWS>
int launch(const W3Args &a, const W3Plan &p, dim3 grid, hipStream_t s) {
  auto kern = k_wgrad3x3<BM, BC, LOGP, ROWS>;
  static bool attr_set = false;  // one process, one GPU: set the LDS opt-in once per instantiation
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            160 * 1024) != hipSuccess)
      return SGH_EUNSUPPORTED;
    attr_set = true;
  }
  SGH_LAUNCH_TIMED(kern, grid, dim3(NT), p.lds, s, a);
  return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
}

}  // namespace

size_t sgh_wgrad3x3_workspace_bytes(const sgh_conv_geom *g) {
  const W3Plan p = plan(g);
  return p.ok ? size_t(p.splits) * 9 * g->K * g->C * sizeof(float) : 0;
}

// Returns SGH_EUNSUPPORTED when the geometry is not covered (the caller then uses the generic path).
int sgh_wgrad3x3_run(const sgh_conv_geom *g, const float *dy, const float *x, float *dW, void *workspace,
                     size_t ws_bytes, hipStream_t s) {
  const W3Plan p = plan(g);
  if (!p.ok) return SGH_EUNSUPPORTED;
  const size_t need = size_t(p.splits) * 9 * g->K * g->C * sizeof(float);
  if (!workspace || ws_bytes < need) return SGH_EWORKSPACE;
  W3Args a;
  a.dy = dy;
  a.x = x;
  a.part = static_cast<float *>(workspace);
  a.N = g->N;
  a.C = g->C;
  a.H = g->H;
  a.W = g->W;
  a.K = g->K;
  a.P = g->P;
  a.Q = g->Q;
  a.ph = g->pad_h;
  a.pw = g->pad_w;
  a.stride = g->stride_h;
  a.RU = p.ru;
  a.units_per_image = p.upi;
  a.total_units = p.total_units;
  a.units_per_split = p.units_per_split;
  a.gx = (g->K + p.bm - 1) / p.bm, a.gy = (g->C + p.bc - 1) / p.bc, a.gz = p.splits;
  a.xcd = sgh_env().conv_xcd_off ? 0 : 1;
  if (long(a.gx) * a.gy * a.gz >= (long(1) << 31)) return SGH_EUNSUPPORTED;
  dim3 grid(unsigned(a.gx * a.gy * a.gz), 1, 1);
  int rc = SGH_EUNSUPPORTED;
  sgh_prof_kernel_begin("conv_wgrad/k_wgrad3x3", 2.0 * g->N * g->K * g->P * g->Q * g->C * 9);
#define W3_CASE(BM_, BC_, LOGP_, ROWS_) \
  if (p.bm == BM_ && p.bc == BC_ && p.logp == LOGP_ && p.rows == ROWS_) rc = launch<BM_, BC_, LOGP_, ROWS_>(a, p, grid, s);
  W3_CASE(128, 32, 6, 3)
  W3_CASE(64, 64, 6, 3)
  W3_CASE(128, 32, 5, 4)
  W3_CASE(64, 64, 5, 4)
  W3_CASE(128, 32, 4, 6)
  W3_CASE(64, 64, 4, 6)
  W3_CASE(128, 32, 4, 9)
  W3_CASE(64, 64, 4, 9)
  W3_CASE(128, 32, 6, 5)
  W3_CASE(128, 32, 5, 9)
  W3_CASE(128, 32, 4, 15)
#undef W3_CASE
  sgh_prof_kernel_end(s);
  if (rc != SGH_OK) return rc;
  // pairs per reduction workgroup: small layers take fewer pairs and more z-lanes per workgroup
  const long kc = long(g->K) * g->C;
  const int cus = sgh_num_cus();
  if (kc / 64 >= cus)
    hipLaunchKernelGGL(k_wgrad3x3_reduce<64>, dim3(int((kc + 63) / 64)), dim3(256), 0, s, a.part, dW, g->K, g->C, p.splits);
  else if (kc / 32 >= cus)
    hipLaunchKernelGGL(k_wgrad3x3_reduce<32>, dim3(int((kc + 31) / 32)), dim3(256), 0, s, a.part, dW, g->K, g->C, p.splits);
  else
    hipLaunchKernelGGL(k_wgrad3x3_reduce<16>, dim3(int((kc + 15) / 16)), dim3(256), 0, s, a.part, dW, g->K, g->C, p.splits);
  return hipGetLastError() == hipSuccess ? SGH_OK : SGH_EINVAL;
}
