// Pooling forward/backward for NCHW fp32.
//
// Max-pool backward is a gather: one thread owns one dx element, visits the (at most
// ceil(kh/sh) * ceil(kw/sw)) windows that contain it in ascending (p, q) order, recomputes each
// window's first maximum (row-major scan, strict '>') and adds dy when the maximum sits on its
// own element.  The additions therefore happen in exactly the order of the CPU scatter loop, so
// dx is bit-identical to it and no atomics are needed.
#include "common.h"
#include "storage.h"

namespace {

constexpr int kBlock = 256;

struct PoolG {
  int H, W, P, Q, kh, kw, sh, sw, ph, pw;
};

// flat index (h * W + w) of the first maximum of window (p, q) in plane `b`; -1 if empty
template <class S>
__device__ __forceinline__ int window_argmax(const typename S::elem *__restrict__ b, const PoolG g, int p, int q,
                                             float *best_out) {
  int hs = p * g.sh - g.ph, ws = q * g.sw - g.pw;
  const int he = min(hs + g.kh, g.H), we = min(ws + g.kw, g.W);
  hs = max(hs, 0);
  ws = max(ws, 0);
  float best = -3.402823466e38f;
  int bi = -1;
  for (int h = hs; h < he; ++h)
    for (int w = ws; w < we; ++w) {
      const float v = S::ld(b + h * g.W + w);
      if (v > best) {
        best = v;
        bi = h * g.W + w;
      }
    }
  if (best_out) *best_out = best;
  return bi;
}

template <class S>
__global__ __launch_bounds__(kBlock) void k_pool_max_fwd(const typename S::elem *__restrict__ x,
                                                        typename S::elem *__restrict__ y, PoolG g, size_t total) {
  const size_t stride = size_t(gridDim.x) * kBlock;
  const int PQ = g.P * g.Q;
  for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < total; i += stride) {
    const size_t plane = i / PQ;
    const int r = int(i - plane * PQ);
    float best;
    window_argmax<S>(x + plane * size_t(g.H) * g.W, g, r / g.Q, r % g.Q, &best);
    S::st(y + i, best);
  }
}

// The residual networks' pooling layer (3 x 3, stride 2, padding 1, even image, Q a multiple of the vector
// length): a thread produces one vector of outputs from two vectors and one element of each of its three input
// rows, comparing in the order of window_argmax (rows top to bottom, columns left to right, strict '>').
template <class S>
__global__ __launch_bounds__(kBlock) void k_pool_max_fwd_3x3s2(const typename S::elem *__restrict__ x,
                                                              typename S::elem *__restrict__ y, int H, int W, size_t nvec) {
  constexpr int V = S::VEC;
  const int P = H >> 1, Q = W >> 1, QV = Q / V;
  const float none = -__builtin_inff();   // (never greater than anything: a position outside the image)
  const size_t stride = size_t(gridDim.x) * kBlock;
  for (size_t iv = size_t(blockIdx.x) * kBlock + threadIdx.x; iv < nvec; iv += stride) {
    const size_t pr = iv / QV;              // plane * P + p
    const int qv = int(iv - pr * QV), q = qv * V;
    const size_t plane = pr / P;
    const int p = int(pr - plane * P);
    const typename S::elem *xb = x + plane * size_t(H) * W;
    float best[V];
#pragma unroll
    for (int j = 0; j < V; ++j) best[j] = -3.402823466e38f;
#pragma unroll
    for (int r = 0; r < 3; ++r) {
      const int h = 2 * p - 1 + r;
      if (h < 0) continue;                  // (h <= H - 1 always: H is even)
      const typename S::elem *row = xb + size_t(h) * W + 2 * q;
      float e[2 * V + 1];
      e[0] = q > 0 ? S::ld(row - 1) : none;
      S::template load16<false>(row, e + 1);
      S::template load16<false>(row + V, e + 1 + V);
#pragma unroll
      for (int j = 0; j < V; ++j)
#pragma unroll
        for (int c = 0; c < 3; ++c)
          if (e[2 * j + c] > best[j]) best[j] = e[2 * j + c];
    }
    S::store16(y + (pr * size_t(Q)) + q, best);
  }
}

template <class S>
__global__ __launch_bounds__(kBlock) void k_pool_max_bwd(const typename S::elem *__restrict__ dy,
                                                        const typename S::elem *__restrict__ x,
                                                        typename S::elem *__restrict__ dx, PoolG g, size_t total) {
  const size_t stride = size_t(gridDim.x) * kBlock;
  const int HW = g.H * g.W, PQ = g.P * g.Q;
  for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < total; i += stride) {
    const size_t plane = i / HW;
    const int r = int(i - plane * HW);
    const int h = r / g.W, w = r - h * g.W;
    const typename S::elem *xb = x + plane * size_t(HW);
    const typename S::elem *db = dy + plane * size_t(PQ);
    // windows p with p*sh - ph <= h < p*sh - ph + kh
    const int hp = h + g.ph, wp = w + g.pw;
    const int p_lo = hp < g.kh ? 0 : (hp - g.kh) / g.sh + 1;
    const int p_hi = min(hp / g.sh, g.P - 1);
    const int q_lo = wp < g.kw ? 0 : (wp - g.kw) / g.sw + 1;
    const int q_hi = min(wp / g.sw, g.Q - 1);
    float s = 0.f;
    for (int p = p_lo; p <= p_hi; ++p)
      for (int q = q_lo; q <= q_hi; ++q)
        if (window_argmax<S>(xb, g, p, q, nullptr) == r) s += S::ld(db + p * g.Q + q);
    S::st(dx + i, s);
  }
}

// Tiled max-pool backward: one workgroup owns a band of TH rows of one (n, c) plane of dx.
//   1. the x rows every window touching the band needs and the dy rows of those windows are
//      staged in LDS (both are contiguous runs of the plane: 128-bit copies when aligned),
//   2. each of those windows gets its first-maximum position (flat h * W + w) into LDS,
//   3. each dx element of the band adds dy over the windows that contain it, in ascending (p, q)
//      order, when the window's maximum sits on it -- the same order as the CPU scatter loop.
// The 256 threads form 64 columns x 4 rows, so no per-element division is needed: a thread's
// column window range is fixed, and the per-row window range is computed once per band row.
// x, dy and dx each cross HBM once (plus the band halo of x).
// KH/KW/SH/SW > 0 fix the window at compile time: the scans are then fully unrolled, every LDS
// read of a window or of a dx element is issued before the first compare, and out-of-range
// positions are predicated instead of branched over.  0 = read the geometry at run time.
template <int KH, int KW, int SH, int SW, class S>
__global__ __launch_bounds__(kBlock) void k_pool_max_bwd_tiled(const typename S::elem *__restrict__ dy,
                                                              const typename S::elem *__restrict__ x,
                                                              typename S::elem *__restrict__ dx, PoolG g, int TH,
                                                              int bands, int max_xrows, int max_np) {
  if (KH > 0) {
    g.kh = KH;
    g.kw = KW;
    g.sh = SH;
    g.sw = SW;
  }
  extern __shared__ float smem[];
  float *xs = smem;                                               // [max_xrows][W]
  float *ds = xs + max_xrows * g.W;                               // [max_np][Q]
  int *widx = reinterpret_cast<int *>(ds + max_np * g.Q);         // [max_np][Q]
  int *prange = widx + max_np * g.Q;                              // [TH][2]: first / last window row of a band row
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int plane = blockIdx.x / bands, band = blockIdx.x - plane * bands;
  const int h0 = band * TH, h1 = min(h0 + TH, g.H);
  // windows p with [p*sh - ph, p*sh - ph + kh) overlapping [h0, h1)
  const int lo_num = h0 + g.ph - g.kh + 1;
  const int p_lo = lo_num <= 0 ? 0 : (lo_num + g.sh - 1) / g.sh;
  const int p_hi = min((h1 - 1 + g.ph) / g.sh, g.P - 1);
  const int np = p_hi - p_lo + 1;
  const int xr0 = max(p_lo * g.sh - g.ph, 0), xr1 = min(p_hi * g.sh - g.ph + g.kh, g.H);  // x rows [xr0, xr1)
  const typename S::elem *xb = x + size_t(plane) * g.H * g.W + xr0 * g.W;
  const typename S::elem *db = dy + size_t(plane) * g.P * g.Q + p_lo * g.Q;
  typename S::elem *ob = dx + size_t(plane) * g.H * g.W;
  const int nx = (xr1 - xr0) * g.W, nd = np > 0 ? np * g.Q : 0;
  // 16 bytes of the storage type per access when the run is aligned (LDS holds floats)
  constexpr int V = S::VEC;
  if ((reinterpret_cast<uintptr_t>(xb) & 15u) == 0 && nx % V == 0) {
#pragma unroll 4
    for (int i = threadIdx.x; i < nx / V; i += kBlock) {
      float v[V];
      S::template load16<false>(xb + i * V, v);
#pragma unroll
      for (int j = 0; j < V; ++j) xs[i * V + j] = v[j];
    }
  } else {
    for (int i = threadIdx.x; i < nx; i += kBlock) xs[i] = S::ld(xb + i);
  }
  for (int i = threadIdx.x; i < nd; i += kBlock) ds[i] = S::ld(db + i);
  for (int i = threadIdx.x; i < h1 - h0; i += kBlock) {
    const int hp = h0 + i + g.ph;
    prange[2 * i] = (hp < g.kh ? 0 : (hp - g.kh) / g.sh + 1) - p_lo;
    prange[2 * i + 1] = min(hp / g.sh, g.P - 1) - p_lo;
  }
  __syncthreads();
  for (int pp = ty; pp < np; pp += 4) {
    const int hs0 = (p_lo + pp) * g.sh - g.ph;
    for (int q = tx; q < g.Q; q += 64) {
      const int ws0 = q * g.sw - g.pw;
      float best = -3.402823466e38f;
      int bi = -1;
      if (KH > 0) {
        float v[KH > 0 ? KH * KW : 1];
#pragma unroll
        for (int dh = 0; dh < KH; ++dh)
#pragma unroll
          for (int dw = 0; dw < KW; ++dw) {
            const int h = hs0 + dh, w = ws0 + dw;
            const bool ok = unsigned(h) < unsigned(g.H) && unsigned(w) < unsigned(g.W);
            const float xv = xs[ok ? (h - xr0) * g.W + w : 0];
            v[dh * KW + dw] = ok ? xv : -3.402823466e38f;
          }
#pragma unroll
        for (int dh = 0; dh < KH; ++dh)
#pragma unroll
          for (int dw = 0; dw < KW; ++dw)
            if (v[dh * KW + dw] > best) {
              best = v[dh * KW + dw];
              bi = (hs0 + dh) * g.W + ws0 + dw;
            }
      } else {
        const int hs = max(hs0, 0), he = min(hs0 + g.kh, g.H);
        const int ws = max(ws0, 0), we = min(ws0 + g.kw, g.W);
        for (int h = hs; h < he; ++h)
          for (int w = ws; w < we; ++w) {
            const float v = xs[(h - xr0) * g.W + w];
            if (v > best) {
              best = v;
              bi = h * g.W + w;
            }
          }
      }
      widx[pp * g.Q + q] = bi;
    }
  }
  __syncthreads();
  if (KH > 0) {
    // A thread owns an SH x SW block of dx.  The windows that can contain any of its elements are
    // NBH x NBW consecutive ones; their arg-max positions and dy values are read once and serve
    // the whole block (a window whose maximum sits on element r necessarily contains r, so
    // testing the position is enough).
    constexpr int SHc = KH > 0 ? SH : 1, SWc = KW > 0 ? SW : 1;
    constexpr int NBH = KH > 0 ? (KH + SH - 2) / SHc + 1 : 1, NBW = KW > 0 ? (KW + SW - 2) / SWc + 1 : 1;
    const int nbh = (h1 - h0 + SHc - 1) / SHc, nbw = (g.W + SWc - 1) / SWc;
    for (int bj = tx; bj < nbw; bj += 64) {
      const int w0 = bj * SWc, wp0 = w0 + g.pw;
      const int ql0 = wp0 < g.kw ? 0 : (wp0 - g.kw) / g.sw + 1;
      for (int bi = ty; bi < nbh; bi += 4) {
        const int hb = h0 + bi * SHc, hp0 = hb + g.ph;
        const int pl0 = (hp0 < g.kh ? 0 : (hp0 - g.kh) / g.sh + 1) - p_lo;
        int wi[NBH * NBW];
        float dv[NBH * NBW];
#pragma unroll
        for (int dp = 0; dp < NBH; ++dp)
#pragma unroll
          for (int dq = 0; dq < NBW; ++dq) {
            const bool ok = pl0 + dp < np && ql0 + dq < g.Q;
            const int o = ok ? (pl0 + dp) * g.Q + ql0 + dq : 0;
            wi[dp * NBW + dq] = ok ? widx[o] : -2;
            dv[dp * NBW + dq] = ds[o];
          }
#pragma unroll
        for (int a = 0; a < SHc; ++a) {
          const int h = hb + a;
          if (h >= h1) break;
          float out[SWc];
#pragma unroll
          for (int b2 = 0; b2 < SWc; ++b2) {
            const int r = h * g.W + w0 + b2;
            // s is never -0.0 (it starts at +0.0), so adding +0.0 for a window that does not match
            // leaves it bit-identical to skipping the addition; ascending (p, q) order as on the CPU
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < NBH * NBW; ++i) s += wi[i] == r ? dv[i] : 0.f;
            out[b2] = s;
          }
          typename S::elem *o = ob + h * g.W + w0;
          if (V == 4 && SWc == 2 && w0 + 1 < g.W && (reinterpret_cast<uintptr_t>(o) & 7u) == 0) {
            typedef float v2f __attribute__((ext_vector_type(2)));
            *reinterpret_cast<v2f *>(o) = v2f{out[0], out[SWc - 1]};
          } else {
#pragma unroll
            for (int b2 = 0; b2 < SWc; ++b2)
              if (w0 + b2 < g.W) S::st(o + b2, out[b2]);
          }
        }
      }
    }
  } else {
    for (int w = tx; w < g.W; w += 64) {
      const int wp = w + g.pw;
      const int ql = wp < g.kw ? 0 : (wp - g.kw) / g.sw + 1;
      const int qh = min(wp / g.sw, g.Q - 1);
      for (int hh = ty; hh < h1 - h0; hh += 4) {
        const int r = (h0 + hh) * g.W + w;
        const int pl = prange[2 * hh], ph_ = prange[2 * hh + 1];
        float s = 0.f;
        for (int p = pl; p <= ph_; ++p)
          for (int q = ql; q <= qh; ++q)
            if (widx[p * g.Q + q] == r) s += ds[p * g.Q + q];
        S::st(ob + r, s);
      }
    }
  }
}

// Max-pool backward for the residual networks' pooling layer: 3 x 3 windows, stride 2, padding 1, even H and W.
// The dx block (rows 2i, 2i+1; columns 2j, 2j+1) can only receive from windows (i, j), (i, j+1), (i+1, j),
// (i+1, j+1), and only at fixed positions of those windows, so instead of tables of arg-max positions and
// dy values in LDS (the general kernel above: 67 vector instructions per dx element, which bound it) a lane
// walks down one window column with everything in registers:
//   * window p shares its top row with window p - 1's bottom row: the per-row first maximum (strict '>',
//     left to right) is computed once per x row, and three of them combine top to bottom -- the same winner
//     as the row-major scan of the CPU loop;
//   * the winner is kept as a code 3 * dh + dw; the right-hand neighbour's code and dy come from lane + 1;
//   * a block's four elements add the dy of the windows whose code names them, in ascending (p, q) order
//     starting from +0.0, exactly the additions of the general kernel.
// A workgroup owns kStripRows block rows per wavefront of one plane; x rows are staged in LDS as stored, behind
// an element and (for the first band) a row of -inf, so no position needs a bounds check.
constexpr int kStripRows = 7;   // block rows per wavefront (a wavefront also computes the window row below them)
constexpr float kLowest = -3.402823466e38f;

struct RowBest {
  float m;
  int k;   // column within the window (0..2), 64 = none
};

template <class S>
__device__ __forceinline__ RowBest row_best(const typename S::elem *row) {   // row -> the window's middle element of one x row
  typedef typename S::elem elem;
  float a, b, c;
  if constexpr (sizeof(elem) == 4) {
    a = row[-1];
    const float2 bc = *reinterpret_cast<const float2 *>(row);
    b = bc.x, c = bc.y;
  } else {
    const unsigned pr = *reinterpret_cast<const unsigned *>(row);
    const elem lo = elem(pr & 0xffffu), hi = elem(pr >> 16);
    a = S::ld(row - 1), b = S::ld(&lo), c = S::ld(&hi);
  }
  RowBest r{kLowest, 64};
  if (a > r.m) r.m = a, r.k = 0;
  if (b > r.m) r.m = b, r.k = 1;
  if (c > r.m) r.m = c, r.k = 2;
  return r;
}

template <class S>
__global__ __launch_bounds__(kBlock) void k_pool_max_bwd_3x3s2(const typename S::elem *__restrict__ dy,
                                                               const typename S::elem *__restrict__ x,
                                                               typename S::elem *__restrict__ dx, int H, int W, int bands) {
  typedef typename S::elem elem;
  constexpr int V = S::VEC;
  typedef sgh_v4u raw;   // 16 bytes: V elements
  // x rows as stored: element (r, w) at (r - r_lo) * pitch + V + w (rows start on 16-byte boundaries), the element
  // before a row and the row above the image hold -inf, which no comparison selects
  extern __shared__ __align__(16) unsigned char xs_raw[];
  elem *xs = reinterpret_cast<elem *>(xs_raw);
  const int P = H >> 1, Q = W >> 1, pitch = W + V;
  const int plane = blockIdx.x / bands, band = blockIdx.x - plane * bands;
  const int i0 = band * (4 * kStripRows), i1 = min(i0 + 4 * kStripRows, P);   // block rows (= window rows) of the band
  const int r_lo = 2 * i0 - 1, r_hi = min(2 * i1 + 1, H - 1), rr0 = max(r_lo, 0);
  const elem *xb = x + size_t(plane) * H * W;
  const elem *db = dy + size_t(plane) * P * Q;
  elem *ob = dx + size_t(plane) * H * W;
  const int vpr = W / V;   // 16-byte (8-byte) vectors per row
  for (int i = threadIdx.x; i < (r_hi - rr0 + 1) * vpr; i += kBlock) {
    const int r = i / vpr, c = (i - r * vpr) * V;
    *reinterpret_cast<raw *>(xs + (rr0 - r_lo + r) * pitch + V + c) =
        __builtin_nontemporal_load(reinterpret_cast<const raw *>(xb + size_t(rr0 + r) * W + c));
  }
  for (int r = threadIdx.x; r <= r_hi - r_lo; r += kBlock) S::st(xs + r * pitch + V - 1, -__builtin_inff());
  if (r_lo < 0)
    for (int c = threadIdx.x; c < pitch; c += kBlock) S::st(xs + c, -__builtin_inff());
  __syncthreads();

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int ia = i0 + wave * kStripRows, ib = min(ia + kStripRows, i1);   // this wavefront's block rows [ia, ib)
  if (ia >= ib) return;
  for (int q0 = 0; q0 < Q; q0 += 63) {   // lanes 0..62 produce blocks, lane 63 only hands its window to lane 62
    const int q = q0 + lane;
    const bool col = q < Q;
    const int qc = col ? q : Q - 1;   // (a lane without a window reads a valid address and discards it)
    float dyr[kStripRows + 1];
#pragma unroll
    for (int k = 0; k <= kStripRows; ++k) {
      const int p = ia + k;
      dyr[k] = (p <= ib && p < P && col) ? S::ld(db + p * Q + q) : 0.f;
    }
    const elem *xq = xs + (2 * ia - r_lo) * pitch + V + 2 * qc;   // element (2 ia, 2 q)
    RowBest top = row_best<S>(xq - pitch);
    int code_p = 64, ncode_p = 64;
    float dy_p = 0.f, ndy_p = 0.f;
#pragma unroll
    for (int k = 0; k <= kStripRows; ++k) {
      const int p = ia + k;
      if (p > ib) break;
      int code = 64;
      if (p < P) {
        const RowBest mid = row_best<S>(xq + (2 * k) * pitch), bot = row_best<S>(xq + (2 * k + 1) * pitch);
        float best = top.m;
        code = top.k;
        if (mid.m > best) best = mid.m, code = 3 + mid.k;
        if (bot.m > best) code = 6 + bot.k;
        if (!col) code = 64;
        top = bot;
      }
      const float dyv = dyr[k];
      const int ncode = __shfl_down(code, 1);
      const float ndy = __shfl_down(dyv, 1);
      if (k > 0 && lane < 63 && col) {
        // block row p - 1: windows (p-1, q), (p-1, q+1), (p, q), (p, q+1) in that order
        const float o00 = 0.f + (code_p == 4 ? dy_p : 0.f);
        const float o01 = (0.f + (code_p == 5 ? dy_p : 0.f)) + (ncode_p == 3 ? ndy_p : 0.f);
        const float o10 = (0.f + (code_p == 7 ? dy_p : 0.f)) + (code == 1 ? dyv : 0.f);
        const float o11 = (((0.f + (code_p == 8 ? dy_p : 0.f)) + (ncode_p == 6 ? ndy_p : 0.f)) + (code == 2 ? dyv : 0.f)) +
                          (ncode == 0 ? ndy : 0.f);
        elem *o = ob + size_t(2 * (p - 1)) * W + 2 * q;
        if constexpr (sizeof(elem) == 4) {
          typedef float v2f __attribute__((ext_vector_type(2)));
          __builtin_nontemporal_store(v2f{o00, o01}, reinterpret_cast<v2f *>(o));
          __builtin_nontemporal_store(v2f{o10, o11}, reinterpret_cast<v2f *>(o + W));
        } else {
          elem t0[2], t1[2];
          S::st(t0, o00), S::st(t0 + 1, o01), S::st(t1, o10), S::st(t1 + 1, o11);
          *reinterpret_cast<unsigned *>(o) = unsigned(t0[0]) | (unsigned(t0[1]) << 16);
          *reinterpret_cast<unsigned *>(o + W) = unsigned(t1[0]) | (unsigned(t1[1]) << 16);
        }
      }
      code_p = code, ncode_p = ncode, dy_p = dyv, ndy_p = ndy;
    }
  }
}

__device__ __forceinline__ int window_count(const PoolG g, int p, int q, int *hs_, int *he_, int *ws_, int *we_) {
  int hs = p * g.sh - g.ph, ws = q * g.sw - g.pw;
  const int he = min(hs + g.kh, g.H), we = min(ws + g.kw, g.W);
  hs = max(hs, 0);
  ws = max(ws, 0);
  *hs_ = hs;
  *he_ = he;
  *ws_ = ws;
  *we_ = we;
  return (he - hs) * (we - ws);  // count-exclude-padding
}

template <class S>
__global__ __launch_bounds__(kBlock) void k_pool_avg_fwd(const typename S::elem *__restrict__ x,
                                                        typename S::elem *__restrict__ y, PoolG g, size_t total) {
  const size_t stride = size_t(gridDim.x) * kBlock;
  const int PQ = g.P * g.Q;
  for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < total; i += stride) {
    const size_t plane = i / PQ;
    const int r = int(i - plane * PQ);
    const typename S::elem *b = x + plane * size_t(g.H) * g.W;
    int hs, he, ws, we;
    const int cnt = window_count(g, r / g.Q, r % g.Q, &hs, &he, &ws, &we);
    float s = 0.f;
    for (int h = hs; h < he; ++h)
      for (int w = ws; w < we; ++w) s += S::ld(b + h * g.W + w);
    S::st(y + i, s / float(cnt));
  }
}

// One window that is the whole plane, planes of at most 64 elements (global average pooling, 7 x 7): a workgroup
// stages its 256 consecutive planes -- one contiguous run of memory -- in LDS with whole-vector loads and a thread
// sums one plane in the order of the loop above.
template <class S>
__global__ __launch_bounds__(kBlock) void k_pool_avg_fwd_global(const typename S::elem *__restrict__ x,
                                                               typename S::elem *__restrict__ y, int HW, size_t planes) {
  constexpr int V = S::VEC;
  extern __shared__ float xs_f[];   // kBlock * HW
  const size_t plane0 = size_t(blockIdx.x) * kBlock;
  const int np = int(planes - plane0 < size_t(kBlock) ? planes - plane0 : size_t(kBlock)), n = np * HW, t = threadIdx.x;
  const typename S::elem *base = x + plane0 * size_t(HW);
  const int nvec = n / V;
  for (int v = t; v < nvec; v += kBlock) {
    float e[V];
    S::template load16<false>(base + v * V, e);
#pragma unroll
    for (int q = 0; q < V; ++q) xs_f[v * V + q] = e[q];
  }
  for (int i = nvec * V + t; i < n; i += kBlock) xs_f[i] = S::ld(base + i);
  __syncthreads();
  if (t < np) {
    float s = 0.f;
    for (int j = 0; j < HW; ++j) s += xs_f[t * HW + j];
    S::st(y + plane0 + t, s / float(HW));
  }
}

template <class S>
__global__ __launch_bounds__(kBlock) void k_pool_avg_bwd(const typename S::elem *__restrict__ dy,
                                                        typename S::elem *__restrict__ dx, PoolG g, size_t total) {
  const size_t stride = size_t(gridDim.x) * kBlock;
  const int HW = g.H * g.W, PQ = g.P * g.Q;
  for (size_t i = size_t(blockIdx.x) * kBlock + threadIdx.x; i < total; i += stride) {
    const size_t plane = i / HW;
    const int r = int(i - plane * HW);
    const int h = r / g.W, w = r - h * g.W;
    const typename S::elem *db = dy + plane * size_t(PQ);
    const int hp = h + g.ph, wp = w + g.pw;
    const int p_lo = hp < g.kh ? 0 : (hp - g.kh) / g.sh + 1;
    const int p_hi = min(hp / g.sh, g.P - 1);
    const int q_lo = wp < g.kw ? 0 : (wp - g.kw) / g.sw + 1;
    const int q_hi = min(wp / g.sw, g.Q - 1);
    float s = 0.f;
    for (int p = p_lo; p <= p_hi; ++p)
      for (int q = q_lo; q <= q_hi; ++q) {
        int hs, he, ws, we;
        const int cnt = window_count(g, p, q, &hs, &he, &ws, &we);
        s += S::ld(db + p * g.Q + q) / float(cnt);
      }
    S::st(dx + i, s);
  }
}

// One window that is the whole plane (global average pooling): every element of a plane receives
// dy[plane] / (H * W), the same arithmetic as the kernel above, written in whole vectors.
template <class S>
__global__ __launch_bounds__(kBlock) void k_pool_avg_bwd_global(const typename S::elem *__restrict__ dy,
                                                               typename S::elem *__restrict__ dx, int HW, size_t total) {
  constexpr int V = S::VEC;
  const size_t stride = size_t(gridDim.x) * kBlock, tid = size_t(blockIdx.x) * kBlock + threadIdx.x;
  const size_t nvec = total / V;
  const float cnt = float(HW);
  for (size_t iv = tid; iv < nvec; iv += stride) {
    const size_t i0 = iv * V;
    size_t plane = i0 / size_t(HW);
    int r = int(i0 - plane * size_t(HW));
    float gv = 0.f + S::ld(dy + plane) / cnt;
    float o[V];
#pragma unroll
    for (int q = 0; q < V; ++q) {
      if (r == HW) {
        r = 0;
        ++plane;
        gv = 0.f + S::ld(dy + plane) / cnt;
      }
      o[q] = gv;
      ++r;
    }
    S::store16(dx + i0, o);
  }
  for (size_t i = nvec * V + tid; i < total; i += stride) S::st(dx + i, 0.f + S::ld(dy + i / size_t(HW)) / cnt);
}

inline int grid_for(size_t n) {
  size_t blocks = (n + kBlock - 1) / kBlock;
  const size_t cap = size_t(sgh_num_cus()) * 32;
  if (blocks > cap) blocks = cap;
  return int(blocks < 1 ? 1 : blocks);
}

inline PoolG to_g(const sgh_pool_geom *g) {
  return PoolG{g->H, g->W, g->P, g->Q, g->kernel_h, g->kernel_w, g->stride_h, g->stride_w, g->pad_h, g->pad_w};
}

inline bool geom_ok(const sgh_pool_geom *g) {
  return g && g->N > 0 && g->C > 0 && g->H > 0 && g->W > 0 && g->kernel_h > 0 && g->kernel_w > 0 && g->stride_h > 0 &&
         g->stride_w > 0 && g->pad_h >= 0 && g->pad_w >= 0 && g->P > 0 && g->Q > 0 &&
         g->P == (g->H + 2 * g->pad_h - g->kernel_h) / g->stride_h + 1 &&
         g->Q == (g->W + 2 * g->pad_w - g->kernel_w) / g->stride_w + 1 &&
         // every window must overlap the image, else a max window would be empty
         g->pad_h < g->kernel_h && g->pad_w < g->kernel_w &&
         size_t(g->H) * g->W < 0x7fffffffu;
}

template <class S>
int pool_fwd(const sgh_pool_geom *g, const typename S::elem *x, typename S::elem *y, void *stream) {
  if (!geom_ok(g) || !x || !y) return SGH_EINVAL;
  const size_t total = size_t(g->N) * g->C * g->P * g->Q;
  if (g->is_max && g->kernel_h == 3 && g->kernel_w == 3 && g->stride_h == 2 && g->stride_w == 2 && g->pad_h == 1 &&
      g->pad_w == 1 && g->H % 2 == 0 && g->W % 2 == 0 && g->Q % S::VEC == 0 && sgh_aligned16(x) && sgh_aligned16(y))
    hipLaunchKernelGGL(k_pool_max_fwd_3x3s2<S>, dim3(grid_for(total / S::VEC)), dim3(kBlock), 0, sgh_stream_of(stream), x, y,
                       g->H, g->W, total / S::VEC);
  else if (g->is_max)
    hipLaunchKernelGGL(k_pool_max_fwd<S>, dim3(grid_for(total)), dim3(kBlock), 0, sgh_stream_of(stream), x, y, to_g(g),
                       total);
  else if (g->P == 1 && g->Q == 1 && g->pad_h == 0 && g->pad_w == 0 && g->kernel_h >= g->H && g->kernel_w >= g->W &&
           g->H * g->W <= 64 && sgh_aligned16(x) && (total + kBlock - 1) / kBlock < 0x7fffffffu)
    hipLaunchKernelGGL(k_pool_avg_fwd_global<S>, dim3(unsigned((total + kBlock - 1) / kBlock)), dim3(kBlock),
                       size_t(kBlock) * g->H * g->W * sizeof(float), sgh_stream_of(stream), x, y, g->H * g->W, total);
  else
    hipLaunchKernelGGL(k_pool_avg_fwd<S>, dim3(grid_for(total)), dim3(kBlock), 0, sgh_stream_of(stream), x, y, to_g(g),
                       total);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

template <class S>
int pool_bwd(const sgh_pool_geom *g, const typename S::elem *dy, const typename S::elem *x, const typename S::elem *y,
             typename S::elem *dx, void *stream) {
  (void)y;
  if (!geom_ok(g) || !dy || !dx) return SGH_EINVAL;
  if (g->is_max && !x) return SGH_EINVAL;
  const size_t total = size_t(g->N) * g->C * g->H * g->W;
  // algorithmic bytes: dy and (max pooling) x in, dx out
  sgh_prof_kernel_scope prof(g->is_max ? "pool_bwd/k_pool_max_bwd" : "pool_bwd/k_pool_avg_bwd",
                      double(sizeof(typename S::elem)) *
                          (double(total) * (g->is_max ? 2 : 1) + double(g->N) * g->C * g->P * g->Q),
                      sgh_stream_of(stream));
  if (g->is_max && g->kernel_h == 3 && g->kernel_w == 3 && g->stride_h == 2 && g->stride_w == 2 && g->pad_h == 1 &&
      g->pad_w == 1 && g->H % 2 == 0 && g->W % S::VEC == 0 && g->W <= 256 &&
      size_t(g->N) * g->C * ((g->H / 2 + 4 * kStripRows - 1) / (4 * kStripRows)) < 0x7fffffffu && sgh_aligned16(x) &&
      sgh_aligned16(dx)) {
    const int bands = (g->H / 2 + 4 * kStripRows - 1) / (4 * kStripRows);
    const size_t lds = size_t(8 * kStripRows + 3) * (g->W + S::VEC) * sizeof(typename S::elem);   // <= 61 KB
    SGH_LAUNCH_TIMED(k_pool_max_bwd_3x3s2<S>, dim3(unsigned(size_t(g->N) * g->C * bands)), dim3(kBlock), lds,
                       sgh_stream_of(stream), dy, x, dx, g->H, g->W, bands);
  } else if (g->is_max) {
    // band height: about 12 KB of x rows per workgroup (measured optimum: enough workgroups per CU to
    // overlap one's staging with another's scans), bands of equal height
    int TH = 3072 / g->W - g->kernel_h;
    if (TH < 1) TH = 1;
    if (TH > g->H) TH = g->H;
    int bands = (g->H + TH - 1) / TH;
    TH = (g->H + bands - 1) / bands;
    bands = (g->H + TH - 1) / TH;
    const int max_np = (TH + g->kernel_h - 2) / g->stride_h + 2;
    const int max_xrows = (max_np - 1) * g->stride_h + g->kernel_h;
    const size_t lds = (size_t(max_xrows) * g->W + size_t(2) * max_np * g->Q + size_t(2) * TH) * sizeof(float);
    const size_t blocks = size_t(g->N) * g->C * bands;
    if (lds <= 48 * 1024 && blocks < 0x7fffffffu && g->W <= 2048) {
      auto kern = k_pool_max_bwd_tiled<0, 0, 0, 0, S>;
      if (g->kernel_h == 3 && g->kernel_w == 3 && g->stride_h == 2 && g->stride_w == 2)
        kern = k_pool_max_bwd_tiled<3, 3, 2, 2, S>;
      else if (g->kernel_h == 2 && g->kernel_w == 2 && g->stride_h == 2 && g->stride_w == 2)
        kern = k_pool_max_bwd_tiled<2, 2, 2, 2, S>;
      else if (g->kernel_h == 3 && g->kernel_w == 3 && g->stride_h == 1 && g->stride_w == 1)
        kern = k_pool_max_bwd_tiled<3, 3, 1, 1, S>;
      SGH_LAUNCH_TIMED(kern, dim3((unsigned)blocks), dim3(kBlock), lds, sgh_stream_of(stream), dy, x, dx, to_g(g), TH,
                         bands, max_xrows, max_np);
    } else {
      SGH_LAUNCH_TIMED(k_pool_max_bwd<S>, dim3(grid_for(total)), dim3(kBlock), 0, sgh_stream_of(stream), dy, x, dx,
                         to_g(g), total);
    }
  } else if (g->P == 1 && g->Q == 1 && g->pad_h == 0 && g->pad_w == 0 && g->kernel_h >= g->H && g->kernel_w >= g->W &&
             sgh_aligned16(dx))
    SGH_LAUNCH_TIMED(k_pool_avg_bwd_global<S>, dim3(grid_for((total + S::VEC - 1) / S::VEC)), dim3(kBlock), 0,
                       sgh_stream_of(stream), dy, dx, g->H * g->W, total);
  else
    SGH_LAUNCH_TIMED(k_pool_avg_bwd<S>, dim3(grid_for(total)), dim3(kBlock), 0, sgh_stream_of(stream), dy, dx, to_g(g),
                       total);
  SGH_LAUNCH_CHECK();
  return SGH_OK;
}

}  // namespace

extern "C" {

int sgh_pool_geom_init(sgh_pool_geom *g, int N, int C, int H, int W, int kernel_h, int kernel_w, int stride_h,
                       int stride_w, int pad_h, int pad_w, int is_max) {
  if (!g) return SGH_EINVAL;
  if (N <= 0 || C <= 0 || H <= 0 || W <= 0 || kernel_h <= 0 || kernel_w <= 0 || stride_h <= 0 || stride_w <= 0 ||
      pad_h < 0 || pad_w < 0)
    return SGH_EINVAL;
  if (H + 2 * pad_h < kernel_h || W + 2 * pad_w < kernel_w) return SGH_EINVAL;
  g->N = N;
  g->C = C;
  g->H = H;
  g->W = W;
  g->kernel_h = kernel_h;
  g->kernel_w = kernel_w;
  g->stride_h = stride_h;
  g->stride_w = stride_w;
  g->pad_h = pad_h;
  g->pad_w = pad_w;
  // PoolingHandle's floor formula (reference: src/model/operation/pooling.cc:48-51)
  g->P = (H + 2 * pad_h - kernel_h) / stride_h + 1;
  g->Q = (W + 2 * pad_w - kernel_w) / stride_w + 1;
  g->is_max = is_max ? 1 : 0;
  return geom_ok(g) ? SGH_OK : SGH_EINVAL;
}

int sgh_pool_fwd_f32(const sgh_pool_geom *g, const float *x, float *y, void *stream) {
  return pool_fwd<StF32>(g, x, y, stream);
}
int sgh_pool_fwd_f16(const sgh_pool_geom *g, const uint16_t *x, uint16_t *y, void *stream) {
  return pool_fwd<StF16>(g, x, y, stream);
}
int sgh_pool_fwd_bf16(const sgh_pool_geom *g, const uint16_t *x, uint16_t *y, void *stream) {
  return pool_fwd<StBF16>(g, x, y, stream);
}
int sgh_pool_bwd_f32(const sgh_pool_geom *g, const float *dy, const float *x, const float *y, float *dx,
                     void *stream) {
  return pool_bwd<StF32>(g, dy, x, y, dx, stream);
}
int sgh_pool_bwd_f16(const sgh_pool_geom *g, const uint16_t *dy, const uint16_t *x, const uint16_t *y, uint16_t *dx,
                     void *stream) {
  return pool_bwd<StF16>(g, dy, x, y, dx, stream);
}
int sgh_pool_bwd_bf16(const sgh_pool_geom *g, const uint16_t *dy, const uint16_t *x, const uint16_t *y, uint16_t *dx,
                      void *stream) {
  return pool_bwd<StBF16>(g, dy, x, y, dx, stream);
}

}  // extern "C"
