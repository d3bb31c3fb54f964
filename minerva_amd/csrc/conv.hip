// Convolution forward, backward-data and backward-filter as implicit GEMMs on the fp32
// MFMA core (gemm_core.h).  Semantics: cuDNN v2 CUDNN_CONVOLUTION (flipped filter),
// zero padding, NCHW / KCRS bytes, as selected by the reference at
// minerva/op/impl/cuda/cuda_perform.cu:227-318:
//   top[n,k,i,j] = bias[k] + sum_{c,r,s} bottom[n,c,i*sv-ph+r,j*sh-pw+s] * filter[k,c,R-1-r,S-1-s]
// With r' = R-1-r, s' = S-1-s the filter is read in its natural order, so it is a plain
// column-major {C*R*S, K} matrix, and the flip moves into the im2col gather.
//
//   forward        : C[(n,i,j), k]      = sum_{(c,r',s')}  im2col(bottom) * filter
//   backward data  : C[(n,y,x), c]      = sum_{(k,r',s')}  gather(top_diff) * filter^T-gather
//   backward filter: C[(c,r',s'), k]    = sum_{(n,i,j)}    gather(bottom) * top_diff   (k range split)
// In every case the GEMM "m" dimension is the one that is contiguous in the output
// tensor, so result stores are coalesced, and no im2col buffer exists in HBM.
// Roofline: fp32 MFMA, 2*N*Ho*Wo*K*C*R*S algorithmic flops per pass.

#include "gemm_core.h"
#include "winograd.h"

namespace {

struct ConvGeom {
  int N, C, K, H, W, Ho, Wo, R, S, ph, pw, sv, sh;
  int HW, HoWo, RS, CRS;
  MnvFastDiv d_RS, d_S, d_HoWo, d_Wo, d_HW, d_W, d_sv, d_sh;
};

#define MNV_FAR (-20000)  // row/col origin that fails every bounds test

__device__ __forceinline__ int pack_yx(int y, int x) { return (y << 16) | (x & 0xffff); }
__device__ __forceinline__ int unpack_y(int p) { return p >> 16; }
__device__ __forceinline__ int unpack_x(int p) { return (int)(short)(p & 0xffff); }

// Every policy comes in two addressing flavours (see the contract in gemm_core.h):
//   FAST   : the reduction index is ordered (filter tap, channel) and a period is one tap,
//            so the im2col offsets and their bounds tests are computed once per tap and a
//            slab of 16 channels only advances a uniform scalar offset.  Needs the channel
//            count of the reduction to be a multiple of 16 (and unit stride for the data
//            gradient).
//   generic: the reduction index is the flat (channel, tap) order, one period per slab.
// The two orders only differ in the order the products are summed.

// ------------------------------------------------------------------ forward
template <bool FAST>
struct ConvFwd {
  static constexpr bool A_KFAST = false, B_KFAST = true;
  static constexpr int A_NOFF = 4, B_NOFF = FAST ? 1 : 4;
  const float* __restrict__ bottom;
  const float* __restrict__ filter;
  const float* __restrict__ bias;
  float* __restrict__ top;
  ConvGeom g;
  int M, N, K, total_slabs, spp;  // GEMM extents: N*Ho*Wo, Kout, C*R*S
  int relu;                       // fused epilogue: top = max(conv + bias, 0)
  struct Res {
    mnv_rsrc a, b;
  };
  struct AState {
    int off[4], yx[4];
  };
  struct BState {};
  __device__ void make_res(Res& r) const {
    r.a = mnv_make_rsrc(bottom, (unsigned)(g.N * g.C * g.HW) * 4u);
    r.b = mnv_make_rsrc(filter, (unsigned)(g.K * g.CRS) * 4u);
  }
  __device__ void a_init(const Res& res, AState& st, int m) const {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      int mm = m + q;
      int img = mnv_fastdiv(mm, g.d_HoWo);
      int pos = mm - img * g.HoWo;
      int i = mnv_fastdiv(pos, g.d_Wo);
      int j = pos - i * g.Wo;
      int y0 = i * g.sv - g.ph, x0 = j * g.sh - g.pw;
      st.off[q] = img * g.C * g.HW + y0 * g.W + x0;
      st.yx[q] = mm < M ? pack_yx(y0, x0) : pack_yx(MNV_FAR, MNV_FAR);
    }
  }
  __device__ void b_init(const Res&, BState&, int) const {}
  __device__ void a_period(const AState& st, unsigned (&off)[4], int, int kl, int period) const {
    int c, rs;
    bool kok = true;
    if (FAST) {  // period = tap, kl = channel within the slab
      rs = period;
      c = kl;
    } else {  // period = slab, flat k = (c, r', s')
      int k = period * 16 + kl;
      kok = k < K;
      c = mnv_fastdiv(k, g.d_RS);
      rs = k - c * g.RS;
    }
    int rp = mnv_fastdiv(rs, g.d_S);
    int sp = rs - rp * g.S;
    int r = g.R - 1 - rp, s = g.S - 1 - sp;  // flipped tap
    int koff = c * g.HW + r * g.W + s;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      int y = unpack_y(st.yx[q]) + r, x = unpack_x(st.yx[q]) + s;
      bool ok = kok & ((unsigned)y < (unsigned)g.H) & ((unsigned)x < (unsigned)g.W);
      off[q] = ok ? (unsigned)(st.off[q] + koff) * 4u : MNV_OOB;
    }
  }
  __device__ void a_load(const Res& r, const AState&, const unsigned (&off)[4], int, int s, int,
                         float (&v)[4]) const {
    mnv_fetch_vec<4>(r.a, off, FAST ? (unsigned)s * 16u * (unsigned)g.HW * 4u : 0u, v);
  }
  size_t extra_lds_bytes() const { return 0; }
  __device__ void block_init(Res&, float*, int, int) const {}
  // generic: `filter` is the caller's tensor [n][c][r'][s'], element (k, n) at n*CRS + k.
  // FAST: `filter` is the permuted copy [n][r's'][c], so the 4 channels of a vector are
  // one 16-byte load and consecutive slabs are consecutive memory.
  __device__ void b_period(const BState&, unsigned (&off)[B_NOFF], int n, int kl,
                           int period) const {
    if (FAST) {
      off[0] = (n < N) ? (unsigned)(n * g.CRS + period * g.C + kl) * 4u : MNV_OOB;
    } else {
#pragma unroll
      for (int q = 0; q < B_NOFF; ++q) {
        int k = period * 16 + kl + q;
        off[q] = ((n < N) & (k < K)) ? (unsigned)(n * K + k) * 4u : MNV_OOB;
      }
    }
  }
  __device__ void b_load(const Res& r, const BState&, const unsigned (&off)[B_NOFF], int, int s,
                         int, float (&v)[4]) const {
    mnv_fetch_vec<B_NOFF>(r.b, off, FAST ? (unsigned)s * 64u : 0u, v);
  }
  // The fused ReLU is the selection mnv_relu_fwd makes on the stored value, so the result has
  // the bits of the two-operator sequence.
  __device__ void c_store(int m, int n, float x) const {
    int img = mnv_fastdiv(m, g.d_HoWo);
    int pos = m - img * g.HoWo;
    float v = x + bias[n];
    if (relu) v = v > 0.f ? v : 0.f;
    top[((size_t)img * N + n) * g.HoWo + pos] = v;
  }
  // four consecutive positions of one channel: one 16-byte store (4-byte aligned) unless the
  // four straddle two images or the end of the batch
  static constexpr bool C_STORE4 = true;
  __device__ void c_store4(int m, int n, const float (&x)[4]) const {
    int img = mnv_fastdiv(m, g.d_HoWo);
    int pos = m - img * g.HoWo;
    if (m + 3 < M && pos + 3 < g.HoWo) {
      const float b = bias[n];
      mnv_f4u v = {x[0] + b, x[1] + b, x[2] + b, x[3] + b};
      if (relu) {
        v.x = v.x > 0.f ? v.x : 0.f; v.y = v.y > 0.f ? v.y : 0.f;
        v.z = v.z > 0.f ? v.z : 0.f; v.w = v.w > 0.f ? v.w : 0.f;
      }
      *reinterpret_cast<mnv_f4u*>(top + ((size_t)img * N + n) * g.HoWo + pos) = v;
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (m + q < M) c_store(m + q, n, x[q]);
    }
  }
};

// Forward without padding (ph == pw == 0, any channel count and stride).  Every tap of
// every output position is a real pixel, so the pixel offset is base(position) + koff(k)
// with koff(k) = ((c*H + R-1-r')*W + S-1-s')*4 for the flat reduction index k = (c, r', s').
// koff is tabulated in LDS once per workgroup; a slab then costs one 16-byte LDS read and
// four adds per vector, and nothing is decomposed or bounds-tested in the main loop.  The
// filter needs no copy: in this order it already is the column-major K x Kout operand.
// Period 0 holds the full slabs, period 1 the last, partial one (masked filter loads).
// A vector is four consecutive k at ONE output position (k-fast): its four loads are 4-byte
// gathers either way, but with four lanes per position a load instruction touches about 20
// cache lines (16 positions, the taps of a vector a few floats apart) where four
// consecutive positions per lane touched 64 at a stride of four pixels -- and conv1
// (stride 4, C = 3) was bound by those L1 look-ups, not by the matrix pipe.
struct ConvFwdNP {
  static constexpr bool A_KFAST = true, B_KFAST = true;
  static constexpr int A_NOFF = 1, B_NOFF = 4;
  const float* __restrict__ bottom;
  const float* __restrict__ filter;
  const float* __restrict__ bias;
  float* __restrict__ top;
  ConvGeom g;
  int M, N, K, total_slabs, spp;  // GEMM extents: N*Ho*Wo, Kout, C*R*S
  int relu;                       // fused epilogue: top = max(conv + bias, 0)
  struct Res {
    mnv_rsrc a, b;
    const unsigned* tab;  // LDS: [total_slabs*16] byte offsets, MNV_OOB past K
  };
  struct AState {};
  struct BState {};
  __device__ void make_res(Res& r) const {
    r.a = mnv_make_rsrc(bottom, (unsigned)(g.N * g.C * g.HW) * 4u);
    r.b = mnv_make_rsrc(filter, (unsigned)(g.K * g.CRS) * 4u);
    r.tab = nullptr;
  }
  size_t extra_lds_bytes() const { return (size_t)total_slabs * 16 * sizeof(unsigned); }
  __device__ void block_init(Res& r, float* extra, int, int) const {
    unsigned* tab = reinterpret_cast<unsigned*>(extra);
    r.tab = tab;
    for (int k = threadIdx.x; k < total_slabs * 16; k += blockDim.x) {
      int c = mnv_fastdiv(k, g.d_RS);
      int rs = k - c * g.RS;
      int rp = mnv_fastdiv(rs, g.d_S), sp = rs - rp * g.S;
      tab[k] = k < K ? (unsigned)(c * g.HW + (g.R - 1 - rp) * g.W + (g.S - 1 - sp)) * 4u : MNV_OOB;
    }
  }
  __device__ void a_init(const Res&, AState&, int) const {}
  __device__ void b_init(const Res&, BState&, int) const {}
  // rows past M are never stored, so they may read any valid pixel
  __device__ void a_period(const AState&, unsigned (&off)[1], int m, int, int) const {
    int mm = m < M ? m : 0;
    int img = mnv_fastdiv(mm, g.d_HoWo);
    int pos = mm - img * g.HoWo;
    int i = mnv_fastdiv(pos, g.d_Wo);
    int j = pos - i * g.Wo;
    off[0] = (unsigned)(img * g.C * g.HW + i * g.sv * g.W + j * g.sh) * 4u;
  }
  // an entry past K is MNV_OOB, and MNV_OOB plus any pixel offset is still out of range
  __device__ void a_load(const Res& r, const AState&, const unsigned (&off)[1], int period, int s,
                         int kl, float (&v)[4]) const {
    typedef unsigned u4 __attribute__((ext_vector_type(4)));
    const u4 t = *reinterpret_cast<const u4*>(
        __builtin_assume_aligned(r.tab + (period * spp + s) * 16 + kl, 16));
#pragma unroll
    for (int q = 0; q < 4; ++q)
      v[q] = __builtin_bit_cast(float,
                                __builtin_amdgcn_raw_buffer_load_b32(r.a, (int)(off[0] + t[q]), 0, 0));
  }
  // filter element (k, n) at n*K + k: four consecutive k are one 16-byte load (4-byte
  // aligned is enough for a buffer load)
  __device__ void b_period(const BState&, unsigned (&off)[4], int n, int kl, int period) const {
    int k = period * spp * 16 + kl;
#pragma unroll
    for (int q = 0; q < 4; ++q)
      off[q] = ((n < N) & (k + q < K)) ? (unsigned)(n * K + k + q) * 4u : MNV_OOB;
  }
  __device__ void b_load(const Res& r, const BState&, const unsigned (&off)[4], int period, int s,
                         int, float (&v)[4]) const {
    if (period == 0 && spp * 16 <= K) {  // uniform: a full slab
      const unsigned one[1] = {off[0]};
      mnv_fetch_vec<1>(r.b, one, (unsigned)s * 64u, v);
    } else {
      mnv_fetch_vec<4>(r.b, off, (unsigned)s * 64u, v);
    }
  }
  __device__ void c_store(int m, int n, float x) const {
    int img = mnv_fastdiv(m, g.d_HoWo);
    int pos = m - img * g.HoWo;
    float v = x + bias[n];
    if (relu) v = v > 0.f ? v : 0.f;
    top[((size_t)img * N + n) * g.HoWo + pos] = v;
  }
  // four consecutive positions of one channel: one 16-byte store (4-byte aligned) unless the
  // four straddle two images or the end of the batch
  static constexpr bool C_STORE4 = true;
  __device__ void c_store4(int m, int n, const float (&x)[4]) const {
    int img = mnv_fastdiv(m, g.d_HoWo);
    int pos = m - img * g.HoWo;
    if (m + 3 < M && pos + 3 < g.HoWo) {
      const float b = bias[n];
      mnv_f4u v = {x[0] + b, x[1] + b, x[2] + b, x[3] + b};
      if (relu) {
        v.x = v.x > 0.f ? v.x : 0.f; v.y = v.y > 0.f ? v.y : 0.f;
        v.z = v.z > 0.f ? v.z : 0.f; v.w = v.w > 0.f ? v.w : 0.f;
      }
      *reinterpret_cast<mnv_f4u*>(top + ((size_t)img * N + n) * g.HoWo + pos) = v;
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (m + q < M) c_store(m + q, n, x[q]);
    }
  }
};

// ------------------------------------------------------------ backward data
// FAST additionally means both strides are 1, so every (row, col) of the shifted window
// is a real output position.
template <bool FAST>
struct ConvBwdData {
  static constexpr bool A_KFAST = false, B_KFAST = true;
  static constexpr int A_NOFF = 4, B_NOFF = FAST ? 1 : 4;
  const float* __restrict__ top_diff;
  const float* __restrict__ filter;
  float* __restrict__ bottom_diff;
  ConvGeom g;
  int M, N, K, total_slabs, spp;  // N*H*W, C, Kout*R*S
  // fused epilogue (or null): the activations the bottom tensor went through a ReLU with;
  // bottom_diff = gate > 0 ? gradient : 0, the selection mnv_relu_bwd makes
  const float* __restrict__ gate;
  struct Res {
    mnv_rsrc a, b;
  };
  struct AState {
    int off[4], yx[4];  // image offset into top_diff; (y+ph-R+1, x+pw-S+1)
  };
  struct BState {};
  __device__ void make_res(Res& r) const {
    r.a = mnv_make_rsrc(top_diff, (unsigned)(g.N * g.K * g.HoWo) * 4u);
    r.b = mnv_make_rsrc(filter, (unsigned)(g.K * g.CRS) * 4u);
  }
  __device__ void a_init(const Res& res, AState& st, int m) const {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      int mm = m + q;
      int img = mnv_fastdiv(mm, g.d_HW);
      int pos = mm - img * g.HW;
      int y = mnv_fastdiv(pos, g.d_W);
      int x = pos - y * g.W;
      int ty0 = y + g.ph - g.R + 1, tx0 = x + g.pw - g.S + 1;
      st.off[q] = img * g.K * g.HoWo + (FAST ? ty0 * g.Wo + tx0 : 0);
      st.yx[q] = mm < M ? pack_yx(ty0, tx0) : pack_yx(MNV_FAR, MNV_FAR);
    }
  }
  __device__ void b_init(const Res&, BState&, int) const {}
  __device__ void a_period(const AState& st, unsigned (&off)[4], int, int kl, int period) const {
    if (FAST) {  // period = tap (r', s'), kl = output channel within the slab
      int rp = mnv_fastdiv(period, g.d_S);
      int sp = period - rp * g.S;
      int koff = kl * g.HoWo + rp * g.Wo + sp;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        int i = unpack_y(st.yx[q]) + rp, j = unpack_x(st.yx[q]) + sp;
        bool ok = ((unsigned)i < (unsigned)g.Ho) & ((unsigned)j < (unsigned)g.Wo);
        off[q] = ok ? (unsigned)(st.off[q] + koff) * 4u : MNV_OOB;
      }
    } else {  // flat k = (ko, r', s')
      int k = period * 16 + kl;
      int ko = mnv_fastdiv(k, g.d_RS);
      int rs = k - ko * g.RS;
      int rp = mnv_fastdiv(rs, g.d_S);
      int sp = rs - rp * g.S;
      int koff = ko * g.HoWo;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        int ty = unpack_y(st.yx[q]) + rp, tx = unpack_x(st.yx[q]) + sp;
        int tyc = ty < 0 ? 0 : ty, txc = tx < 0 ? 0 : tx;
        int i = mnv_fastdiv(tyc, g.d_sv), j = mnv_fastdiv(txc, g.d_sh);
        bool ok = (k < K) & (ty >= 0) & (tx >= 0) & (i * g.sv == ty) & (j * g.sh == tx) &
                  (i < g.Ho) & (j < g.Wo);
        off[q] = ok ? (unsigned)(st.off[q] + koff + i * g.Wo + j) * 4u : MNV_OOB;
      }
    }
  }
  __device__ void a_load(const Res& r, const AState&, const unsigned (&off)[4], int, int s, int,
                         float (&v)[4]) const {
    mnv_fetch_vec<4>(r.a, off, FAST ? (unsigned)s * 16u * (unsigned)g.HoWo * 4u : 0u, v);
  }
  size_t extra_lds_bytes() const { return 0; }
  __device__ void block_init(Res&, float*, int, int) const {}
  // B[kk, c] = filter[ko, c, r', s'].  FAST reads the permuted copy [c][r's'][ko].
  __device__ void b_period(const BState&, unsigned (&off)[B_NOFF], int n, int kl,
                           int period) const {
    if (FAST) {
      off[0] = (n < N) ? (unsigned)((n * g.RS + period) * g.K + kl) * 4u : MNV_OOB;
    } else {
      int k = period * 16 + kl;
      int ko = mnv_fastdiv(k, g.d_RS);
      int rs = k - ko * g.RS;
#pragma unroll
      for (int q = 0; q < B_NOFF; ++q) {
        bool ok = (n < N) & (k + q < K);
        off[q] = ok ? (unsigned)(ko * g.CRS + n * g.RS + rs) * 4u : MNV_OOB;
        ++rs;
        bool wrap = rs == g.RS;
        rs = wrap ? 0 : rs;
        ko += wrap ? 1 : 0;
      }
    }
  }
  __device__ void b_load(const Res& r, const BState&, const unsigned (&off)[B_NOFF], int, int s,
                         int, float (&v)[4]) const {
    mnv_fetch_vec<B_NOFF>(r.b, off, FAST ? (unsigned)s * 64u : 0u, v);
  }
  __device__ void c_store(int m, int n, float x) const {
    int img = mnv_fastdiv(m, g.d_HW);
    int pos = m - img * g.HW;
    const size_t at = ((size_t)img * N + n) * g.HW + pos;
    if (gate) x = gate[at] > 0.f ? x : 0.f;
    bottom_diff[at] = x;
  }
  static constexpr bool C_STORE4 = true;
  __device__ void c_store4(int m, int n, const float (&x)[4]) const {
    int img = mnv_fastdiv(m, g.d_HW);
    int pos = m - img * g.HW;
    if (m + 3 < M && pos + 3 < g.HW) {
      const size_t at = ((size_t)img * N + n) * g.HW + pos;
      mnv_f4u v = {x[0], x[1], x[2], x[3]};
      if (gate) {
        const mnv_f4u t = *reinterpret_cast<const mnv_f4u*>(gate + at);
        v.x = t.x > 0.f ? v.x : 0.f; v.y = t.y > 0.f ? v.y : 0.f;
        v.z = t.z > 0.f ? v.z : 0.f; v.w = t.w > 0.f ? v.w : 0.f;
      }
      *reinterpret_cast<mnv_f4u*>(bottom_diff + at) = v;
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (m + q < M) c_store(m + q, n, x[q]);
    }
  }
};

// ---------------------------------------------------------- backward filter
struct ConvBwdFilter {
  static constexpr bool A_KFAST = true, B_KFAST = true;
  static constexpr int A_NOFF = 4, B_NOFF = 4;
  const float* __restrict__ bottom;
  const float* __restrict__ top_diff;
  float* __restrict__ filter_diff;
  ConvGeom g;
  int M, N, K, total_slabs, spp;  // C*R*S, Kout, N*Ho*Wo
  int accumulate;                 // filter_diff += (a later chunk of images)
  // Parameter update in the store: filter_diff receives sgd_w - sgd_scale * gradient
  // (sgd_w may be filter_diff itself)
  const float* sgd_w;
  float sgd_scale;
  struct Res {
    mnv_rsrc a, b;
  };
  struct AState {
    int off, dyx;  // c*H*W + dy*W + dx ; (dy, dx) = (R-1-r'-ph, S-1-s'-pw)
  };
  struct BState {};
  __device__ void make_res(Res& r) const {
    r.a = mnv_make_rsrc(bottom, (unsigned)(g.N * g.C * g.HW) * 4u);
    r.b = mnv_make_rsrc(top_diff, (unsigned)(g.N * g.K * g.HoWo) * 4u);
  }
  __device__ void a_init(const Res& res, AState& st, int m) const {
    int c = mnv_fastdiv(m, g.d_RS);
    int rs = m - c * g.RS;
    int rp = mnv_fastdiv(rs, g.d_S);
    int sp = rs - rp * g.S;
    int dy = g.R - 1 - rp - g.ph, dx = g.S - 1 - sp - g.pw;
    st.off = c * g.HW + dy * g.W + dx;
    st.dyx = m < M ? pack_yx(dy, dx) : pack_yx(MNV_FAR, MNV_FAR);
  }
  __device__ void b_init(const Res&, BState&, int) const {}
  // A[m, kk..kk+3] = bottom[img, c, i*sv + dy, j*sh + dx] for kk = (img, i, j)
  __device__ void a_period(const AState& st, unsigned (&off)[4], int, int kl, int period) const {
    int k = period * 16 + kl;
    int img = mnv_fastdiv(k, g.d_HoWo);
    int pos = k - img * g.HoWo;
    int i = mnv_fastdiv(pos, g.d_Wo);
    int j = pos - i * g.Wo;
    const int dy = unpack_y(st.dyx), dx = unpack_x(st.dyx);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      int y = i * g.sv + dy, x = j * g.sh + dx;
      bool ok = (k + q < K) & ((unsigned)y < (unsigned)g.H) & ((unsigned)x < (unsigned)g.W);
      unsigned o = (unsigned)(img * g.C * g.HW + st.off + i * g.sv * g.W + j * g.sh) * 4u;
      off[q] = ok ? o : MNV_OOB;
      ++j;
      bool wj = j == g.Wo;
      j = wj ? 0 : j;
      i += wj ? 1 : 0;
      bool wi = i == g.Ho;
      i = wi ? 0 : i;
      img += wi ? 1 : 0;
    }
  }
  __device__ void a_load(const Res& r, const AState&, const unsigned (&off)[4], int, int, int,
                         float (&v)[4]) const {
    mnv_fetch_vec<4>(r.a, off, 0u, v);
  }
  size_t extra_lds_bytes() const { return 0; }
  __device__ void block_init(Res&, float*, int, int) const {}
  // B[kk..kk+3, ko] = top_diff[img, ko, i, j]
  __device__ void b_period(const BState&, unsigned (&off)[4], int n, int kl, int period) const {
    int k = period * 16 + kl;
    int img = mnv_fastdiv(k, g.d_HoWo);
    int pos = k - img * g.HoWo;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      bool ok = (n < N) & (k + q < K);
      off[q] = ok ? (unsigned)((img * N + n) * g.HoWo + pos) * 4u : MNV_OOB;
      ++pos;
      bool wrap = pos == g.HoWo;
      pos = wrap ? 0 : pos;
      img += wrap ? 1 : 0;
    }
  }
  __device__ void b_load(const Res& r, const BState&, const unsigned (&off)[4], int, int, int,
                         float (&v)[4]) const {
    mnv_fetch_vec<4>(r.b, off, 0u, v);
  }
  __device__ void c_store(int m, int n, float x) const {
    const size_t at = (size_t)n * M + m;
    if (sgd_w) x = sgd_w[at] - sgd_scale * x;
    else if (accumulate) x = filter_diff[at] + x;
    filter_diff[at] = x;
  }
};

// Filter gradient, fast addressing.  The GEMM rows are ordered (tap, channel) instead of
// (channel, tap), so a thread's tap is fixed and the only thing that changes from slab to
// slab is which 16 output positions are reduced.  The reduction runs image by image
// (one period per image, positions padded to a multiple of 16).  A workgroup first writes,
// for every tap its rows touch, a table pos -> byte offset of the input pixel that the tap
// pairs with output position pos (or MNV_OOB when that pixel is padding or pos is past the
// image); a slab's im2col offsets are then one 16-byte LDS read and four adds per vector.
// top_diff is read with 16-byte loads of 4 consecutive positions; only the last, partial
// slab of an image needs per-element masking.
//
// NP ("no padding", any channel count): with ph == pw == 0 every tap of every output
// position is a real pixel, so the pixel offset splits into a row part (channel, tap) and a
// position part: one position table serves all rows, which stay in (channel, tap) order.
//
// LK (padded convolutions whose channel count is a multiple of 16, so that every 16 rows of
// a tile are 16 consecutive channels of one tap): the gathered operand is fetched with the
// slab's 16 positions on 16 consecutive lanes.  A load instruction then reads 64 contiguous
// bytes of each of four channel planes instead of 16 bytes of each of sixteen; a thread's
// eight rows are 16 rows apart, so what distinguishes them (tap, first channel) is uniform
// and lives in the workgroup's Res; and nothing else changes: same tile in LDS, same
// products, same order.  LK = 1: all rows of a tile share one tap (channel counts that are
// multiples of 128: one table entry and one add per thread and slab); LK = 2: a table entry
// per row group; LK = 3: the rows of a tile lie in at most two taps (96 channels: conv2 of the
// AlexNet shape), so a thread reads two table entries per slab and every row group picks one
// of the two by a uniform flag.  Row groups past M fetch whatever their offsets point at: their
// accumulators are never stored.
template <bool NP, int LK = 0>
struct ConvBwdFilterFast {
  static constexpr bool A_KFAST = true, B_KFAST = true;
  static constexpr bool A_LANE_K = LK != 0;
  static constexpr int A_NOFF = 1, B_NOFF = 1;
  const float* __restrict__ bottom;
  const float* __restrict__ top_diff;
  float* __restrict__ filter_diff;
  ConvGeom g;
  int M, N, K, total_slabs, spp;  // C*R*S rows in (tap, c) order, Kout, N*Ho*Wo
  int PP, taps_per_block;         // padded positions per image, table rows per workgroup
  MnvFastDiv d_C;
  int accumulate;                 // filter_diff += (a later chunk of images)
  const float* sgd_w;             // update in the store, as in ConvBwdFilter
  float sgd_scale;
  struct Res {
    mnv_rsrc a, b;
    const unsigned* tab;  // LDS: [taps_per_block][PP]
    int tap0;             // first tap of the workgroup's rows
    // LK: row group j (rows m0 + 16 j ...) starts at channel c0: c0 * H * W * 4, its table
    // row (tap - tap0) * PP, and whether it lies inside M
    unsigned group_off[LK ? 8 : 1];
    int group_trow[LK ? 8 : 1];
    bool group_ok[LK ? 8 : 1];
    bool group_second[LK ? 8 : 1];  // LK = 3: the group's rows lie in the tile's second tap
  };
  struct AState {
    unsigned cbase;  // c*H*W*4, or MNV_OOB for rows past M
    int trow;        // (tap - first tap of the workgroup) * PP
  };
  struct BState {};
  __device__ void make_res(Res& r) const {
    r.a = mnv_make_rsrc(bottom, (unsigned)(g.N * g.C * g.HW) * 4u);
    r.b = mnv_make_rsrc(top_diff, (unsigned)(g.N * g.K * g.HoWo) * 4u);
    r.tab = nullptr;
    r.tap0 = 0;
  }
  size_t extra_lds_bytes() const { return (size_t)taps_per_block * PP * sizeof(unsigned); }
  __device__ void block_init(Res& r, float* extra, int m0, int) const {
    unsigned* tab = reinterpret_cast<unsigned*>(extra);
    r.tab = tab;
    const int tap0 = mnv_fastdiv(m0, d_C);
    r.tap0 = tap0;
    if (LK) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int row = m0 + 16 * j, tap = mnv_fastdiv(row, d_C);
        r.group_off[j] = (unsigned)((row - tap * g.C) * g.HW) * 4u;
        r.group_trow[j] = (tap - tap0 < taps_per_block ? tap - tap0 : 0) * PP;
        r.group_ok[j] = row < M;
        r.group_second[j] = tap - tap0 == 1;
      }
    }
    for (int e = threadIdx.x; e < taps_per_block * PP; e += blockDim.x) {
      int t = e / PP, pos = e - t * PP;
      int tap = tap0 + t;
      int rp = mnv_fastdiv(tap, g.d_S), sp = tap - rp * g.S;
      int dy = NP ? 0 : g.R - 1 - rp - g.ph, dx = NP ? 0 : g.S - 1 - sp - g.pw;
      int i = mnv_fastdiv(pos, g.d_Wo), j = pos - i * g.Wo;
      int y = i * g.sv + dy, x = j * g.sh + dx;
      bool ok = (pos < g.HoWo) & (NP | (tap < g.RS)) & ((unsigned)y < (unsigned)g.H) &
                ((unsigned)x < (unsigned)g.W);
      tab[e] = ok ? (unsigned)(y * g.W + x) * 4u : MNV_OOB;
    }
  }
  __device__ void a_init(const Res& res, AState& st, int m) const {
    if (NP) {  // m = (c, r', s'); the tap's shift is part of the row offset
      int c = mnv_fastdiv(m, g.d_RS);
      int rs = m - c * g.RS;
      int rp = mnv_fastdiv(rs, g.d_S), sp = rs - rp * g.S;
      st.cbase = m < M ? (unsigned)(c * g.HW + (g.R - 1 - rp) * g.W + (g.S - 1 - sp)) * 4u : MNV_OOB;
      st.trow = 0;
      return;
    }
    if (LK) {  // the thread's row inside its groups of 16: a channel offset
      st.cbase = (unsigned)((m & 15) * g.HW) * 4u;
      st.trow = 0;
      return;
    }
    int tap = mnv_fastdiv(m, d_C);
    int c = m - tap * g.C;
    st.cbase = m < M ? (unsigned)(c * g.HW) * 4u : MNV_OOB;
    int t = tap - res.tap0;
    st.trow = (t < taps_per_block ? t : 0) * PP;  // rows past M read a valid table row; cbase masks them
  }
  __device__ void b_init(const Res&, BState&, int) const {}
  // off[0]: byte offset of the vector's entries of slab 0 in the table (the pixel offsets
  // come from the table every slab); a slab then adds s * 64 to it, one instruction
  __device__ void a_period(const AState& st, unsigned (&off)[1], int, int kl, int) const {
    off[0] = (unsigned)(st.trow + kl) * 4u;
  }
  template <int AV>
  __device__ void a_load_lanek(const Res& r, const AState& st, int period, int s, int kl,
                               float (&v)[AV][4]) const {
    static_assert(AV * 4 <= 8, "row groups of a tile");
    const unsigned img = (unsigned)period * (unsigned)(g.C * g.HW) * 4u;
    const int pos = s * 16 + kl;
    const unsigned one = st.cbase + r.tab[pos];
    const unsigned two = LK == 3 ? st.cbase + r.tab[PP + pos] : 0u;
#pragma unroll
    for (int j = 0; j < AV * 4; ++j) {
      unsigned voff = one;
      if (LK == 3) voff = r.group_second[j] ? two : one;
      if (LK == 2) {
        voff = st.cbase + r.tab[r.group_trow[j] + pos];
        voff = r.group_ok[j] ? voff : MNV_OOB;
      }
      v[j / 4][j % 4] = __builtin_bit_cast(
          float, __builtin_amdgcn_raw_buffer_load_b32(r.a, (int)voff, (int)(img + r.group_off[j]), 0));
    }
  }
  __device__ void a_load(const Res& r, const AState& st, const unsigned (&off)[1], int period, int s,
                         int, float (&v)[4]) const {
    // the four entries are one aligned 16-byte LDS read: rows are PP (a multiple of 16)
    // entries long and kl is a multiple of 4
    typedef unsigned u4 __attribute__((ext_vector_type(4)));
    const u4 t = *reinterpret_cast<const u4*>(__builtin_assume_aligned(
        reinterpret_cast<const char*>(r.tab) + (off[0] + (unsigned)s * 64u), 16));
    const unsigned soff = (unsigned)period * (unsigned)(g.C * g.HW) * 4u;
#pragma unroll
    for (int q = 0; q < 4; ++q)
      v[q] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                           r.a, (int)(st.cbase + t[q]), (int)soff, 0));
  }
  __device__ void b_period(const BState&, unsigned (&off)[1], int n, int kl, int) const {
    off[0] = n < N ? (unsigned)(n * g.HoWo + kl) * 4u : MNV_OOB;
  }
  // Every slab is one 16-byte load per vector.  In the last slab of an image the positions
  // past the image read whatever follows in memory (the next plane, or 0 past the tensor);
  // b_stash_fix zeroes them on their way to LDS, when the values have arrived anyway.  (A
  // branch to per-element loads at this point made the wavefront wait for every load in
  // flight, the gathered operand's just-issued ones included, once per image.)
  static constexpr bool B_STASH_FIX = true;
  __device__ void b_load(const Res& r, const BState&, const unsigned (&off)[1], int period, int s,
                         int, float (&v)[4]) const {
    const unsigned soff = ((unsigned)period * (unsigned)(g.K * g.HoWo) + (unsigned)s * 16u) * 4u;
    mnv_fetch_vec<1>(r.b, off, soff, v);
  }
  __device__ void b_stash_fix(int s, int kl, float (&v)[4]) const {
    if (s * 16 + 16 > g.HoWo) {  // uniform
      const int first = s * 16 + kl;
#pragma unroll
      for (int q = 0; q < 4; ++q) v[q] = first + q < g.HoWo ? v[q] : 0.f;
    }
  }
  __device__ void c_store(int m, int n, float x) const {
    int row = m;
    if (!NP) {
      int tap = mnv_fastdiv(m, d_C);
      row = (m - tap * g.C) * g.RS + tap;
    }
    const size_t at = (size_t)n * M + row;
    if (sgd_w) x = sgd_w[at] - sgd_scale * x;
    else if (accumulate) x = filter_diff[at] + x;
    filter_diff[at] = x;
  }
};

// Filter permutations for the FAST policies (a few MB at most, one pass):
//   to_rsc: out[k][r's'][c] = in[k][c][r's']      (forward)
//   to_crk: out[c][r's'][k] = in[k][c][r's']      (data gradient)
__global__ __launch_bounds__(256) void mnv_filter_permute_kernel(const float* __restrict__ in,
                                                                 float* __restrict__ out, int K,
                                                                 int C, int RS, bool to_crk) {
  const int total = K * C * RS;
  for (int o = blockIdx.x * 256 + threadIdx.x; o < total; o += gridDim.x * 256) {
    int k, c, rs;
    if (to_crk) {
      k = o % K;
      rs = (o / K) % RS;
      c = o / (K * RS);
    } else {
      c = o % C;
      rs = (o / C) % RS;
      k = o / (C * RS);
    }
    out[o] = in[(k * C + c) * RS + rs];
  }
}

int permute_filter(const float* in, float* out, int K, int C, int RS, bool to_crk, hipStream_t s) {
  int total = K * C * RS;
  int blocks = (total + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(mnv_filter_permute_kernel, dim3(blocks), dim3(256), 0, s, in, out, K, C, RS,
                     to_crk);
  return MNV_LAUNCH_STATUS();
}

typedef MnvGemmTile<128, 128, 16, 2, 2> TileBig;
typedef MnvGemmTile<64, 64, 16, 2, 2> TileSmall;
typedef MnvGemmTile<128, 128, 16, 4, 1, 0, 96> Tile96;  // four wavefronts of 32 x 96
// Four wavefronts of 32 x 32 for outputs of at most 32 columns (a convolution with few
// output channels): a 64-column tile would spend half or more of its multiplies on padding.
// 64 columns are staged because a slab of 32 would not give every thread a vector to fetch.
typedef MnvGemmTile<128, 64, 16, 4, 1, 0, 32> TileThin;

// tile 0: 64x64 output tiles, tile 1: 128x128, tile 2: 128x96, tile 3: 128x32
// Eight wavefronts of 64 x 64 (512 threads, two workgroups per CU): a quarter fewer bytes
// fetched and staged per multiply than TileBig, and every element summed in the same order.
// For the (tap, channel) forward and data-gradient policies, when the 256 x 128 tiles fill
// the chip's two-per-CU slots in whole rounds to 97% (conv3 / conv4 forward and conv4 / conv5
// data gradient of the AlexNet shape at batch 256: 507 tiles on 512 slots, 2-3% faster; conv2
// forward, 1458 tiles in three rounds of 512 at 95%, is 3% SLOWER than on 128 x 128 tiles with
// their cut tail).
typedef MnvGemmTile<256, 128, 16, 4, 2> TileTall;
template <class P>
int launch_tile(int tile, const P& p, int splits, void* ws, hipStream_t s, size_t tail_bytes = 0) {
  if constexpr (P::A_KFAST == false && P::B_NOFF == 1) {
    if (tile == 1 && splits == 1) {
      const long long tiles = (long long)((p.M + 255) / 256) * ((p.N + 127) / 128);
      const long long slots = 2LL * mnv_cu_count(), rounds = (tiles + slots - 1) / slots;
      if ((double)p.M * p.N >= 0.97 * (double)(rounds * slots) * 256.0 * 128.0)
        return mnv_gemm_launch<TileTall>(p, 1, ws, s);
    }
  }
  switch (tile) {
    case 0: return mnv_gemm_launch<TileSmall>(p, splits, ws, s);
    case 2: return mnv_gemm_launch<Tile96>(p, splits, ws, s, tail_bytes);
    case 3: return mnv_gemm_launch<TileThin>(p, splits, ws, s);
    default: return mnv_gemm_launch<TileBig>(p, splits, ws, s, tail_bytes);
  }
}
const int kTileM[4] = {64, 128, 128, 128}, kTileN[4] = {64, 128, 96, 32};

// The filter gradient: few output tiles and a very long k.  On the large tiles it runs as
// one launch of as many workgroups as the chip holds, every one with the same number of
// k-slabs (stream-k: aligned k ranges of every tile, the rest in shares; see mnv_gemm_kernel),
// when the workspace holds the partial tiles; otherwise, and on the small tiles, in `splits`
// whole k ranges.
// Slabs the filter gradient's loads run ahead (see mnv_gemm_kernel): two, which costs a
// fourth workgroup per CU.  Measured on the four padded convolutions of the AlexNet shape
// with the aligned plan: one slab ahead and four workgroups per CU 3.88 ms over the four
// launches, two ahead and three per CU 3.84 ms.
#ifndef MNV_SK_PF
#define MNV_SK_PF 2
#endif
// `plan` (optional): nothing is launched; plan[0] = rows of the tile, plan[1] = k ranges,
// plan[2] = workgroups of the stream-k launch (0: k ranges).
template <class P>
int launch_filter_gradient(int tile, const P& p, int splits, void* ws, size_t ws_bytes, hipStream_t s,
                           int* plan = nullptr) {
  if (plan) {
    plan[0] = kTileM[tile];
    plan[1] = splits;
    plan[2] = 0;
  }
  if (tile == 1 || tile == 2) {
    bool done = false;
    int* wgs = plan ? plan + 2 : nullptr;
    const int rc = tile == 1 ? mnv_gemm_streamk_launch<TileBig, MNV_SK_PF>(p, ws, ws_bytes, s, &done, wgs)
                             : mnv_gemm_streamk_launch<Tile96, MNV_SK_PF>(p, ws, ws_bytes, s, &done, wgs);
    if (rc || done) {
      if (plan && done) plan[1] = 1;
      return rc;
    }
  }
  if (plan) return MNV_OK;
  return launch_tile(tile, p, splits, ws, s);
}

// Bytes the large tiles' launches want for the partial tiles of a cut tail (0: no tail).
size_t tail_workspace_bytes(int tile, int m, int n, int slabs) {
  if (tile != 1 && tile != 2) return 0;
  const long long tiles = (long long)((m + kTileM[tile] - 1) / kTileM[tile]) * ((n + kTileN[tile] - 1) / kTileN[tile]);
  const size_t tile_floats = (size_t)kTileM[tile] * kTileN[tile];
  const MnvTailPlan t = mnv_tail_plan(tiles, slabs, tile_floats, (size_t)-1 / sizeof(float));
  return t.z > 1 ? (size_t)(tiles - t.begin) * t.z * tile_floats * sizeof(float) : 0;
}

// 128-row tiles: 96 columns wide when that leaves clearly fewer idle columns than 128
// (an output 96 or 192 wide), since the narrower tile does a little less work per byte
// staged.
int wide_tile(int n) {
  int pad128 = (n + 127) / 128 * 128, pad96 = (n + 95) / 96 * 96;
  return pad96 * 10 < pad128 * 9 ? 2 : 1;
}

int make_geom(ConvGeom* g, int N, int C, int K, int H, int W, int ph, int pw, int sv, int sh,
              int R, int S) {
  if (N <= 0 || C <= 0 || K <= 0 || H <= 0 || W <= 0 || ph < 0 || pw < 0 || sv <= 0 ||
      sh <= 0 || R <= 0 || S <= 0)
    return MNV_ERR_INVALID;
  int Ho = (H + 2 * ph - R) / sv + 1, Wo = (W + 2 * pw - S) / sh + 1;
  if (H + 2 * ph < R || W + 2 * pw < S || Ho <= 0 || Wo <= 0) return MNV_ERR_INVALID;
  // 16-bit packed coordinates and 32-bit element offsets
  if (H + ph + R >= 16000 || W + pw + S >= 16000) return MNV_ERR_INVALID;
  const long long lim = (1LL << 29) - 1;  // 32-bit byte offsets into each tensor
  if ((long long)N * C * H * W > lim || (long long)N * K * Ho * Wo > lim ||
      (long long)K * C * R * S > lim)
    return MNV_ERR_INVALID;
  g->N = N; g->C = C; g->K = K; g->H = H; g->W = W; g->Ho = Ho; g->Wo = Wo;
  g->R = R; g->S = S; g->ph = ph; g->pw = pw; g->sv = sv; g->sh = sh;
  g->HW = H * W; g->HoWo = Ho * Wo; g->RS = R * S; g->CRS = C * R * S;
  g->d_RS = mnv_fastdiv_make(g->RS);
  g->d_S = mnv_fastdiv_make(S);
  g->d_HoWo = mnv_fastdiv_make(g->HoWo);
  g->d_Wo = mnv_fastdiv_make(Wo);
  g->d_HW = mnv_fastdiv_make(g->HW);
  g->d_W = mnv_fastdiv_make(W);
  g->d_sv = mnv_fastdiv_make(sv);
  g->d_sh = mnv_fastdiv_make(sh);
  return MNV_OK;
}

// Images per launch: bottom, top and filter are read through 32-bit byte offsets, so one
// launch takes at most 2^29 - 1 elements of each.  A larger batch (up to the reference's
// limit of 2^31 - 1 elements per tensor) runs as several launches over chunks of images --
// images are the slowest dimension, so a chunk is a contiguous slice of bottom and top --
// with the filter gradient accumulated chunk by chunk.  0: a single image (or the filter)
// is too large.
int images_per_launch(int N, int C, int K, int H, int W, int ph, int pw, int sv, int sh, int R, int S) {
  if (N <= 0 || C <= 0 || K <= 0 || H <= 0 || W <= 0 || ph < 0 || pw < 0 || sv <= 0 || sh <= 0 ||
      R <= 0 || S <= 0 || H + 2 * ph < R || W + 2 * pw < S)
    return 0;
  const long long lim = (1LL << 29) - 1;
  const long long Ho = (H + 2 * ph - R) / sv + 1, Wo = (W + 2 * pw - S) / sh + 1;
  const long long per_bottom = (long long)C * H * W, per_top = (long long)K * Ho * Wo;
  if ((long long)K * C * R * S > lim || per_bottom > lim || per_top > lim) return 0;
  if (per_bottom * N > 0x7fffffffLL || per_top * N > 0x7fffffffLL) return 0;
  long long chunk = lim / (per_bottom > per_top ? per_bottom : per_top);
  return (int)(chunk < N ? chunk : N);
}

int pick_tile(int m, int n) {
  if (n <= 32) return 3;
  long long big = (long long)((m + 127) / 128) * ((n + 127) / 128);
  if (big < 128 || m <= 64 || n <= 64) return 0;
  return wide_tile(n);
}

// A 64x64 or 128x32 tile does little arithmetic per k-slab, so a slab costs one trip to
// memory and back; its kernels need about 64 registers and at most 24 KB of LDS, which
// lets a CU hold six to eight workgroups whose trips overlap.  When the output has fewer tiles than that, the
// reduction is cut into k ranges (at least six slabs each) until about eight workgroups per
// CU are in flight.  `ws_floats`: workspace left for the partial results.
int small_tile_splits(int tile, int m, int n, int slabs, size_t ws_floats) {
  if (tile != 0 && tile != 3) return 1;
  const int bm = kTileM[tile], bn = kTileN[tile];
  long long tiles = (long long)((m + bm - 1) / bm) * ((n + bn - 1) / bn);
  const long long cus = mnv_cu_count();
  if (tiles >= 6 * cus) return 1;
  long long want = (8 * cus + tiles - 1) / tiles;
  if (want > slabs / 6) want = slabs / 6;
  size_t fit = ws_floats / ((size_t)m * n);
  if ((size_t)want > fit) want = (long long)fit;
  return want < 2 ? 1 : (int)want;
}

// Workspace layout of the forward and data-gradient convolutions: the permuted filter
// (when the fast policy applies) first, then, 256-byte aligned, the partial results.
size_t align256(size_t bytes) { return (bytes + 255) & ~(size_t)255; }

// k ranges of the filter gradient: up to 256, and up to 512 for outputs of at most 16384
// elements, whose partial results cost next to nothing (the MNIST CNN's filters: its step
// 0.28 -> 0.25 ms; conv1 of the AlexNet shape with 341 ranges instead of 255: 0.50 -> 0.54 ms).
#define MNV_BWDF_MAX_SPLITS 256
#define MNV_BWDF_MAX_SPLITS_SMALL 512

// The filter gradient gets its parallelism from splitting the long N*Ho*Wo reduction,
// so it keeps the 128x128 tile (twice the operand reuse) unless the output is tiny.
int bwd_filter_tile(int m, int n) {
  if (n <= 32) return 3;
  return (m <= 64 || n <= 64) ? 0 : wide_tile(n);
}

int bwd_filter_splits(int m, int n, int k, size_t ws_floats) {
  const int tile = bwd_filter_tile(m, n);
  const int bm = kTileM[tile], bn = kTileN[tile];
  long long tiles = (long long)((m + bm - 1) / bm) * ((n + bn - 1) / bn);
  int slabs = (k + 15) / 16;
  int max_splits = (size_t)m * n <= 16384 ? MNV_BWDF_MAX_SPLITS_SMALL : MNV_BWDF_MAX_SPLITS;
  if (max_splits > slabs / 8) max_splits = slabs / 8;
  size_t fit = ws_floats / ((size_t)m * n);
  if ((size_t)max_splits > fit) max_splits = (int)fit;
  return mnv_pick_splits(tiles, slabs, max_splits);
}

}  // namespace

extern "C" {

size_t mnv_conv_fwd_workspace_bytes(int N, int C, int K, int H, int W, int ph, int pw, int sv,
                                   int sh, int R, int S) {
  ConvGeom g;
  if (make_geom(&g, N, C, K, H, W, ph, pw, sv, sh, R, S)) return 0;
  const size_t permuted = C % 16 == 0 ? (size_t)K * g.CRS * sizeof(float) : 0;
  const int gm = N * g.HoWo, gn = K;
  const int splits = small_tile_splits(pick_tile(gm, gn), gm, gn, (g.CRS + 15) / 16, (size_t)-1);
  const size_t tail = tail_workspace_bytes(pick_tile(gm, gn), gm, gn, (g.CRS + 15) / 16);
  size_t need = tail ? align256(permuted) + tail
                     : splits > 1 ? align256(permuted) + (size_t)splits * gm * gn * sizeof(float) : permuted;
  if (mnv_wino_images(N, C, K, H, W, ph, pw, R, S, sv, sh, (size_t)-1)) {
    const size_t w = mnv_wino_workspace_bytes(N, C, K, H, W, ph, pw, R);
    if (w > need) need = w;
  }
  return need;
}

static int conv_fwd_impl(const float* bottom, const float* filter, const float* bias, float* top,
                         int N, int C, int K, int H, int W, int ph, int pw, int sv, int sh, int R,
                         int S, void* workspace, size_t workspace_bytes, mnv_stream_t stream,
                         int relu) {
  ConvGeom g;
  if (!bottom || !filter || !bias || !top) return MNV_ERR_INVALID;
  int rc = make_geom(&g, N, C, K, H, W, ph, pw, sv, sh, R, S);
  if (rc) return rc;
  int gm = N * g.HoWo, gn = K, gk = g.CRS;
  hipStream_t s = mnv_stream(stream);
  // 3 x 3 and 5 x 5 unit-stride layers with enough channels and tiles: minimal filtering, see
  // winograd.hip (its transformed tensors are read and written in 16-byte vectors)
  if (const int images = mnv_wino_images(N, C, K, H, W, ph, pw, R, S, sv, sh,
                                         workspace && mnv_aligned16(workspace) ? workspace_bytes : 0))
    return mnv_wino_conv(bottom, filter, bias, nullptr, top, N, C, K, H, W, ph, pw, R, 0, relu, images,
                         workspace, workspace_bytes, s);
  const int tile = pick_tile(gm, gn);
  const size_t permuted_bytes = (size_t)K * g.CRS * sizeof(float);
  // the no-padding policy reads the filter where it is; for a small problem the extra
  // launch that permutes the filter for the fast policy would cost more than it gains
  const bool np = ph == 0 && pw == 0 && gk <= 4096;
  const bool fast = C % 16 == 0 && workspace && workspace_bytes >= permuted_bytes &&
                    !(np && (tile == 0 || tile == 3));
  // what is left of the workspace after the permuted filter holds the partial results
  const size_t used = fast ? align256(permuted_bytes) : 0;
  float* part = workspace && workspace_bytes > used ? reinterpret_cast<float*>(static_cast<char*>(workspace) + used) : nullptr;
  const int splits = small_tile_splits(tile, gm, gn, (gk + 15) / 16,
                                       part ? (workspace_bytes - used) / sizeof(float) : 0);
  if (fast) {
    float* wp = static_cast<float*>(workspace);
    rc = permute_filter(filter, wp, K, C, g.RS, false, s);
    if (rc) return rc;
    ConvFwd<true> p{bottom, wp, bias, top, g, gm, gn, gk, g.RS * (C / 16), C / 16, relu};
    return launch_tile(tile, p, splits, part, s, part ? workspace_bytes - used : 0);
  }
  if (np) {
    ConvFwdNP p{bottom, filter, bias, top, g, gm, gn, gk, (gk + 15) / 16, gk >= 16 ? gk / 16 : 1, relu};
    return launch_tile(tile, p, splits, part, s, part ? workspace_bytes - used : 0);
  }
  ConvFwd<false> p{bottom, filter, bias, top, g, gm, gn, gk, (gk + 15) / 16, 1, relu};
  return launch_tile(tile, p, splits, part, s, part ? workspace_bytes - used : 0);
}

static int conv_fwd_chunks(const float* bottom, const float* filter, const float* bias, float* top,
                           int N, int C, int K, int H, int W, int ph, int pw, int sv, int sh, int R,
                           int S, void* workspace, size_t workspace_bytes, mnv_stream_t stream,
                           int relu) {
  const int chunk = images_per_launch(N, C, K, H, W, ph, pw, sv, sh, R, S);
  if (chunk <= 0 || chunk >= N)  // the usual case, and invalid geometry (refused inside)
    return conv_fwd_impl(bottom, filter, bias, top, N, C, K, H, W, ph, pw, sv, sh, R, S, workspace,
                         workspace_bytes, stream, relu);
  if (!bottom || !top) return MNV_ERR_INVALID;
  const size_t per_bottom = (size_t)C * H * W;
  const size_t per_top = (size_t)K * ((H + 2 * ph - R) / sv + 1) * ((W + 2 * pw - S) / sh + 1);
  for (int n0 = 0; n0 < N; n0 += chunk) {
    const int nn = N - n0 < chunk ? N - n0 : chunk;
    int rc = conv_fwd_impl(bottom + n0 * per_bottom, filter, bias, top + n0 * per_top, nn, C, K, H,
                           W, ph, pw, sv, sh, R, S, workspace, workspace_bytes, stream, relu);
    if (rc) return rc;
  }
  return MNV_OK;
}

int mnv_conv_fwd(const float* bottom, const float* filter, const float* bias, float* top, int N,
                 int C, int K, int H, int W, int ph, int pw, int sv, int sh, int R, int S,
                 void* workspace, size_t workspace_bytes, mnv_stream_t stream) {
  return conv_fwd_chunks(bottom, filter, bias, top, N, C, K, H, W, ph, pw, sv, sh, R, S, workspace,
                         workspace_bytes, stream, 0);
}

int mnv_conv_fwd_relu(const float* bottom, const float* filter, const float* bias, float* top,
                      int N, int C, int K, int H, int W, int ph, int pw, int sv, int sh, int R,
                      int S, void* workspace, size_t workspace_bytes, mnv_stream_t stream) {
  return conv_fwd_chunks(bottom, filter, bias, top, N, C, K, H, W, ph, pw, sv, sh, R, S, workspace,
                         workspace_bytes, stream, 1);
}

size_t mnv_conv_bwd_data_workspace_bytes(int N, int C, int K, int H, int W, int ph, int pw,
                                        int sv, int sh, int R, int S) {
  ConvGeom g;
  if (make_geom(&g, N, C, K, H, W, ph, pw, sv, sh, R, S)) return 0;
  const size_t permuted = (sv == 1 && sh == 1 && K % 16 == 0) ? (size_t)K * g.CRS * sizeof(float) : 0;
  const int gm = N * g.HW, gn = C;
  const int splits = small_tile_splits(pick_tile(gm, gn), gm, gn, (K * g.RS + 15) / 16, (size_t)-1);
  const size_t tail = tail_workspace_bytes(pick_tile(gm, gn), gm, gn, (K * g.RS + 15) / 16);
  size_t need = tail ? align256(permuted) + tail
                     : splits > 1 ? align256(permuted) + (size_t)splits * gm * gn * sizeof(float) : permuted;
  if (mnv_wino_images(N, K, C, g.Ho, g.Wo, R - 1 - ph, S - 1 - pw, R, S, sv, sh, (size_t)-1)) {
    const size_t w = mnv_wino_workspace_bytes(N, K, C, g.Ho, g.Wo, R - 1 - ph, S - 1 - pw, R);
    if (w > need) need = w;
  }
  return need;
}

static int conv_bwd_data_impl(const float* top_diff, const float* filter, const float* gate,
                              float* bottom_diff, int N, int C, int K, int H, int W, int ph,
                              int pw, int sv, int sh, int R, int S, void* workspace,
                              size_t workspace_bytes, mnv_stream_t stream) {
  ConvGeom g;
  if (!top_diff || !filter || !bottom_diff) return MNV_ERR_INVALID;
  int rc = make_geom(&g, N, C, K, H, W, ph, pw, sv, sh, R, S);
  if (rc) return rc;
  int gm = N * g.HW, gn = C, gk = K * g.RS;
  hipStream_t s = mnv_stream(stream);
  // the same correlation, of top_diff with the unflipped filters, under a padding of R - 1 - pad
  if (const int images = mnv_wino_images(N, K, C, g.Ho, g.Wo, R - 1 - ph, S - 1 - pw, R, S, sv, sh,
                                         workspace && mnv_aligned16(workspace) ? workspace_bytes : 0))
    return mnv_wino_conv(top_diff, filter, nullptr, gate, bottom_diff, N, K, C, g.Ho, g.Wo, R - 1 - ph,
                         S - 1 - pw, R, 1, 0, images, workspace, workspace_bytes, s);
  const int tile = pick_tile(gm, gn);
  const size_t permuted_bytes = (size_t)K * g.CRS * sizeof(float);
  const bool fast = sv == 1 && sh == 1 && K % 16 == 0 && workspace && workspace_bytes >= permuted_bytes;
  const size_t used = fast ? align256(permuted_bytes) : 0;
  float* part = workspace && workspace_bytes > used ? reinterpret_cast<float*>(static_cast<char*>(workspace) + used) : nullptr;
  const int splits = small_tile_splits(tile, gm, gn, (gk + 15) / 16,
                                       part ? (workspace_bytes - used) / sizeof(float) : 0);
  if (fast) {
    float* wq = static_cast<float*>(workspace);
    rc = permute_filter(filter, wq, K, C, g.RS, true, s);
    if (rc) return rc;
    ConvBwdData<true> p{top_diff, wq, bottom_diff, g, gm, gn, gk, g.RS * (K / 16), K / 16, gate};
    return launch_tile(tile, p, splits, part, s, part ? workspace_bytes - used : 0);
  }
  ConvBwdData<false> p{top_diff, filter, bottom_diff, g, gm, gn, gk, (gk + 15) / 16, 1, gate};
  return launch_tile(tile, p, splits, part, s, part ? workspace_bytes - used : 0);
}

static int conv_bwd_data_chunks(const float* top_diff, const float* filter, const float* gate,
                                float* bottom_diff, int N, int C, int K, int H, int W, int ph,
                                int pw, int sv, int sh, int R, int S, void* workspace,
                                size_t workspace_bytes, mnv_stream_t stream) {
  const int chunk = images_per_launch(N, C, K, H, W, ph, pw, sv, sh, R, S);
  if (chunk <= 0 || chunk >= N)
    return conv_bwd_data_impl(top_diff, filter, gate, bottom_diff, N, C, K, H, W, ph, pw, sv, sh, R,
                              S, workspace, workspace_bytes, stream);
  if (!top_diff || !bottom_diff) return MNV_ERR_INVALID;
  const size_t per_bottom = (size_t)C * H * W;
  const size_t per_top = (size_t)K * ((H + 2 * ph - R) / sv + 1) * ((W + 2 * pw - S) / sh + 1);
  for (int n0 = 0; n0 < N; n0 += chunk) {
    const int nn = N - n0 < chunk ? N - n0 : chunk;
    int rc = conv_bwd_data_impl(top_diff + n0 * per_top, filter, gate ? gate + n0 * per_bottom : nullptr,
                                bottom_diff + n0 * per_bottom, nn, C, K, H, W, ph, pw, sv, sh, R, S,
                                workspace, workspace_bytes, stream);
    if (rc) return rc;
  }
  return MNV_OK;
}

int mnv_conv_bwd_data(const float* top_diff, const float* filter, float* bottom_diff, int N,
                      int C, int K, int H, int W, int ph, int pw, int sv, int sh, int R, int S,
                      void* workspace, size_t workspace_bytes, mnv_stream_t stream) {
  return conv_bwd_data_chunks(top_diff, filter, nullptr, bottom_diff, N, C, K, H, W, ph, pw, sv, sh,
                              R, S, workspace, workspace_bytes, stream);
}

int mnv_conv_bwd_data_relu(const float* top_diff, const float* filter, const float* bottom,
                           float* bottom_diff, int N, int C, int K, int H, int W, int ph, int pw,
                           int sv, int sh, int R, int S, void* workspace, size_t workspace_bytes,
                           mnv_stream_t stream) {
  if (!bottom) return MNV_ERR_INVALID;
  return conv_bwd_data_chunks(top_diff, filter, bottom, bottom_diff, N, C, K, H, W, ph, pw, sv, sh,
                              R, S, workspace, workspace_bytes, stream);
}

size_t mnv_conv_bwd_filter_workspace_bytes(int N, int C, int K, int H, int W, int ph, int pw,
                                           int sv, int sh, int R, int S) {
  ConvGeom g;
  if (make_geom(&g, N, C, K, H, W, ph, pw, sv, sh, R, S)) return 0;
  int splits = bwd_filter_splits(g.CRS, K, N * g.HoWo, (size_t)-1);
  size_t bytes = splits > 1 ? (size_t)splits * g.CRS * K * sizeof(float) : 0;
  // the stream-k plan of the large tiles: at most four workgroups per CU, a partial tile each
  // and one more per output tile
  const int tile = bwd_filter_tile(g.CRS, K);
  if (tile == 1 || tile == 2) {
    const long long tiles = (long long)((g.CRS + kTileM[tile] - 1) / kTileM[tile]) *
                            ((K + kTileN[tile] - 1) / kTileN[tile]);
    const size_t sk = (size_t)(4 * mnv_cu_count() + tiles) * kTileM[tile] * kTileN[tile] * sizeof(float);
    if (tiles <= 4LL * mnv_cu_count() && sk > bytes) bytes = sk;
  }
  if (mnv_wino_grad_images(N, C, K, H, W, ph, pw, R, S, sv, sh, (size_t)-1)) {
    const size_t w = mnv_wino_grad_workspace_bytes(N, C, K, H, W, ph, pw, R);
    if (w > bytes) bytes = w;
  }
  return bytes;
}

static int conv_bwd_filter_impl(const float* bottom, const float* top_diff, float* filter_diff,
                                int N, int C, int K, int H, int W, int ph, int pw, int sv, int sh,
                                int R, int S, void* workspace, size_t workspace_bytes,
                                mnv_stream_t stream, int accumulate,
                                const float* sgd_w = nullptr, float sgd_scale = 0.f,
                                int* plan = nullptr) {
  ConvGeom g;
  if (!plan && (!bottom || !top_diff || !filter_diff)) return MNV_ERR_INVALID;
  int rc = make_geom(&g, N, C, K, H, W, ph, pw, sv, sh, R, S);
  if (rc) return rc;
  int gm = g.CRS, gn = K, gk = N * g.HoWo;
  hipStream_t s = mnv_stream(stream);
  // 3 x 3 and 5 x 5 unit-stride layers with enough channels and tiles: minimal filtering of the
  // filter gradient, F(r x r, m x m), see winograd.hip
  if (const int images = mnv_wino_grad_images(N, C, K, H, W, ph, pw, R, S, sv, sh,
                                              workspace && (plan || mnv_aligned16(workspace)) ? workspace_bytes : 0))
    return mnv_wino_filter_grad(bottom, top_diff, filter_diff, N, C, K, H, W, ph, pw, R, images,
                                accumulate, sgd_w, sgd_scale, workspace, workspace_bytes, s, plan);
  int splits = bwd_filter_splits(gm, gn, gk, workspace ? workspace_bytes / sizeof(float) : 0);
  const int tile = bwd_filter_tile(gm, gn);
  // Fast addressing: rows in (tap, channel) order with per-tap offset tables in LDS.  The
  // tables of all taps a 128-row tile touches must fit beside the tiles.
  const int PP = (g.HoWo + 15) / 16 * 16;
  // Taps whose rows meet one 128-row tile, over all tiles (rows are in (tap, channel) order
  // and tiles start at multiples of 128): 1 when 128 divides C, 2 for C = 96, never more than
  // (128 + C - 1) / C + 1.  Sized exactly, conv2's tables (C = 96, 27 x 27 positions) take
  // 5.9 KB instead of 8.8 KB, which is what lets four workgroups share a CU's 160 KB of LDS.
  int taps_per_block = 1;
  for (int m0 = 0; m0 < gm; m0 += 128) {
    const int last = (m0 + 127 < gm ? m0 + 127 : gm - 1) / C;
    if (last - m0 / C + 1 > taps_per_block) taps_per_block = last - m0 / C + 1;
    if (m0 / 128 >= C) break;  // the pattern of m0 % C repeats after C tiles
  }
  if (tile != 0 && ph == 0 && pw == 0 && (size_t)PP * 4 <= 24 * 1024) {
    ConvBwdFilterFast<true> p{bottom, top_diff, filter_diff, g, gm, gn, gk, N * (PP / 16),
                              PP / 16, PP, 1, mnv_fastdiv_make(C), accumulate, sgd_w, sgd_scale};
    return launch_filter_gradient(tile, p, splits, workspace, workspace_bytes, s, plan);
  }
  if (tile != 0 && C % 128 == 0 && (size_t)PP * 4 <= 24 * 1024) {
    ConvBwdFilterFast<false, 1> p{bottom, top_diff, filter_diff, g, gm, gn, gk, N * (PP / 16),
                                  PP / 16, PP, 1, mnv_fastdiv_make(C), accumulate, sgd_w, sgd_scale};
    return launch_filter_gradient(tile, p, splits, workspace, workspace_bytes, s, plan);
  }
  if (tile != 0 && C % 16 == 0 && taps_per_block == 2 && (size_t)taps_per_block * PP * 4 <= 24 * 1024) {
    ConvBwdFilterFast<false, 3> p{bottom, top_diff, filter_diff, g, gm, gn, gk, N * (PP / 16),
                                  PP / 16, PP, taps_per_block, mnv_fastdiv_make(C), accumulate,
                                  sgd_w, sgd_scale};
    return launch_filter_gradient(tile, p, splits, workspace, workspace_bytes, s, plan);
  }
  if (tile != 0 && C % 16 == 0 && (size_t)taps_per_block * PP * 4 <= 24 * 1024) {
    ConvBwdFilterFast<false, 2> p{bottom, top_diff, filter_diff, g, gm, gn, gk, N * (PP / 16),
                                  PP / 16, PP, taps_per_block, mnv_fastdiv_make(C), accumulate,
                                  sgd_w, sgd_scale};
    return launch_filter_gradient(tile, p, splits, workspace, workspace_bytes, s, plan);
  }
  if (tile != 0 && (size_t)taps_per_block * PP * 4 <= 24 * 1024) {
    ConvBwdFilterFast<false> p{bottom, top_diff, filter_diff, g, gm, gn, gk, N * (PP / 16),
                               PP / 16, PP, taps_per_block, mnv_fastdiv_make(C), accumulate, sgd_w, sgd_scale};
    return launch_filter_gradient(tile, p, splits, workspace, workspace_bytes, s, plan);
  }
  ConvBwdFilter p{bottom, top_diff, filter_diff, g, gm, gn, gk, (gk + 15) / 16, 1, accumulate, sgd_w, sgd_scale};
  return launch_filter_gradient(tile, p, splits, workspace, workspace_bytes, s, plan);
}

int mnv_conv_bwd_filter(const float* bottom, const float* top_diff, float* filter_diff, int N,
                        int C, int K, int H, int W, int ph, int pw, int sv, int sh, int R, int S,
                        void* workspace, size_t workspace_bytes, mnv_stream_t stream) {
  const int chunk = images_per_launch(N, C, K, H, W, ph, pw, sv, sh, R, S);
  if (chunk <= 0 || chunk >= N)
    return conv_bwd_filter_impl(bottom, top_diff, filter_diff, N, C, K, H, W, ph, pw, sv, sh, R, S,
                                workspace, workspace_bytes, stream, 0);
  if (!bottom || !top_diff) return MNV_ERR_INVALID;
  const size_t per_bottom = (size_t)C * H * W;
  const size_t per_top = (size_t)K * ((H + 2 * ph - R) / sv + 1) * ((W + 2 * pw - S) / sh + 1);
  for (int n0 = 0; n0 < N; n0 += chunk) {
    const int nn = N - n0 < chunk ? N - n0 : chunk;
    int rc = conv_bwd_filter_impl(bottom + n0 * per_bottom, top_diff + n0 * per_top, filter_diff, nn,
                                  C, K, H, W, ph, pw, sv, sh, R, S, workspace, workspace_bytes,
                                  stream, n0 > 0);
    if (rc) return rc;
  }
  return MNV_OK;
}

int mnv_conv_bwd_filter_plan(int N, int C, int K, int H, int W, int ph, int pw, int sv, int sh, int R,
                             int S, size_t workspace_bytes, int* tile_rows, int* k_ranges,
                             int* streamk_workgroups) {
  int plan[3] = {0, 0, 0};
  const int chunk = images_per_launch(N, C, K, H, W, ph, pw, sv, sh, R, S);
  if (chunk <= 0) return MNV_ERR_INVALID;
  // the workspace is only compared with sizes here, never dereferenced
  void* some = workspace_bytes ? reinterpret_cast<void*>(&plan) : nullptr;
  int rc = conv_bwd_filter_impl(nullptr, nullptr, nullptr, chunk < N ? chunk : N, C, K, H, W, ph, pw, sv,
                                sh, R, S, some, workspace_bytes, nullptr, 0, nullptr, 0.f, plan);
  if (rc) return rc;
  if (tile_rows) *tile_rows = plan[0];
  if (k_ranges) *k_ranges = plan[1];
  if (streamk_workgroups) *streamk_workgroups = plan[2];
  return MNV_OK;
}

int mnv_conv_bwd_filter_sgd(const float* bottom, const float* top_diff, const float* filter,
                            float scale, float* filter_out, int N, int C, int K, int H, int W,
                            int ph, int pw, int sv, int sh, int R, int S, void* workspace,
                            size_t workspace_bytes, mnv_stream_t stream) {
  if (!filter || !filter_out) return MNV_ERR_INVALID;
  // a gradient summed over several launches cannot be folded into the store of one
  const int chunk = images_per_launch(N, C, K, H, W, ph, pw, sv, sh, R, S);
  if (chunk > 0 && chunk < N) return MNV_ERR_INVALID;
  return conv_bwd_filter_impl(bottom, top_diff, filter_out, N, C, K, H, W, ph, pw, sv, sh, R, S,
                              workspace, workspace_bytes, stream, 0, filter, scale);
}

}  // extern "C"
