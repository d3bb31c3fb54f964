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

// ------------------------------------------------------------------ forward
template <bool VECB>
struct ConvFwd {
  static constexpr bool A_KFAST = false, B_KFAST = true;
  const float* __restrict__ bottom;
  const float* __restrict__ filter;
  const float* __restrict__ bias;
  float* __restrict__ top;
  ConvGeom g;
  int M, N, K;  // GEMM extents: N*Ho*Wo, Kout, C*R*S
  struct AState {
    int off[4], yx[4];
  };
  struct BState {};
  __device__ void a_init(AState& st, int m) const {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      int mm = m + q;
      if (mm < M) {
        int img = mnv_fastdiv(mm, g.d_HoWo);
        int pos = mm - img * g.HoWo;
        int i = mnv_fastdiv(pos, g.d_Wo);
        int j = pos - i * g.Wo;
        int y0 = i * g.sv - g.ph, x0 = j * g.sh - g.pw;
        st.off[q] = img * g.C * g.HW + y0 * g.W + x0;
        st.yx[q] = pack_yx(y0, x0);
      } else {
        st.off[q] = 0;
        st.yx[q] = pack_yx(MNV_FAR, MNV_FAR);
      }
    }
  }
  __device__ void b_init(BState&, int) const {}
  __device__ void a_fetch(const AState& st, int, int k, float (&v)[4]) const {
    if (k >= K) {
      v[0] = v[1] = v[2] = v[3] = 0.f;
      return;
    }
    int c = mnv_fastdiv(k, g.d_RS);
    int rs = k - c * g.RS;
    int rp = mnv_fastdiv(rs, g.d_S);
    int sp = rs - rp * g.S;
    int r = g.R - 1 - rp, s = g.S - 1 - sp;  // flipped tap
    int koff = c * g.HW + r * g.W + s;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      int y = unpack_y(st.yx[q]) + r, x = unpack_x(st.yx[q]) + s;
      bool ok = (unsigned)y < (unsigned)g.H && (unsigned)x < (unsigned)g.W;
      v[q] = ok ? bottom[st.off[q] + koff] : 0.f;
    }
  }
  __device__ void b_fetch(const BState&, int n, int k, float (&v)[4]) const {
    if (VECB) {
      if (n < N && k < K) {
        mnv_f4 t = *reinterpret_cast<const mnv_f4*>(filter + (size_t)n * K + k);
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
      } else {
        v[0] = v[1] = v[2] = v[3] = 0.f;
      }
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q) v[q] = (n < N && k + q < K) ? filter[(size_t)n * K + k + q] : 0.f;
    }
  }
  __device__ void c_store(int m, int n, float x) const {
    int img = mnv_fastdiv(m, g.d_HoWo);
    int pos = m - img * g.HoWo;
    top[((size_t)img * N + n) * g.HoWo + pos] = x + bias[n];
  }
};

// ------------------------------------------------------------ backward data
struct ConvBwdData {
  static constexpr bool A_KFAST = false, B_KFAST = true;
  const float* __restrict__ top_diff;
  const float* __restrict__ filter;
  float* __restrict__ bottom_diff;
  ConvGeom g;
  int M, N, K;  // N*H*W, C, Kout*R*S
  struct AState {
    int off[4], yx[4];  // image offset into top_diff; (y+ph-R+1, x+pw-S+1)
  };
  struct BState {};
  __device__ void a_init(AState& st, int m) const {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      int mm = m + q;
      if (mm < M) {
        int img = mnv_fastdiv(mm, g.d_HW);
        int pos = mm - img * g.HW;
        int y = mnv_fastdiv(pos, g.d_W);
        int x = pos - y * g.W;
        st.off[q] = img * g.K * g.HoWo;
        st.yx[q] = pack_yx(y + g.ph - g.R + 1, x + g.pw - g.S + 1);
      } else {
        st.off[q] = 0;
        st.yx[q] = pack_yx(MNV_FAR, MNV_FAR);
      }
    }
  }
  __device__ void b_init(BState&, int) const {}
  __device__ void a_fetch(const AState& st, int, int k, float (&v)[4]) const {
    if (k >= K) {
      v[0] = v[1] = v[2] = v[3] = 0.f;
      return;
    }
    int ko = mnv_fastdiv(k, g.d_RS);
    int rs = k - ko * g.RS;
    int rp = mnv_fastdiv(rs, g.d_S);
    int sp = rs - rp * g.S;
    int koff = ko * g.HoWo;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      int ty = unpack_y(st.yx[q]) + rp, tx = unpack_x(st.yx[q]) + sp;
      float val = 0.f;
      if (ty >= 0 && tx >= 0) {
        int i = mnv_fastdiv(ty, g.d_sv), j = mnv_fastdiv(tx, g.d_sh);
        if (i * g.sv == ty && j * g.sh == tx && i < g.Ho && j < g.Wo)
          val = top_diff[st.off[q] + koff + i * g.Wo + j];
      }
      v[q] = val;
    }
  }
  // B[kk, c] = filter[ko, c, r', s'] for kk = (ko, r', s')
  __device__ void b_fetch(const BState&, int n, int k, float (&v)[4]) const {
    int ko = mnv_fastdiv(k, g.d_RS);
    int rs = k - ko * g.RS;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      v[q] = (n < N && k + q < K) ? filter[(size_t)ko * g.CRS + n * g.RS + rs] : 0.f;
      if (++rs == g.RS) {
        rs = 0;
        ++ko;
      }
    }
  }
  __device__ void c_store(int m, int n, float x) const {
    int img = mnv_fastdiv(m, g.d_HW);
    int pos = m - img * g.HW;
    bottom_diff[((size_t)img * N + n) * g.HW + pos] = x;
  }
};

// ---------------------------------------------------------- backward filter
struct ConvBwdFilter {
  static constexpr bool A_KFAST = true, B_KFAST = true;
  const float* __restrict__ bottom;
  const float* __restrict__ top_diff;
  float* __restrict__ filter_diff;
  ConvGeom g;
  int M, N, K;  // C*R*S, Kout, N*Ho*Wo
  struct AState {
    int off, dyx;  // c*H*W + dy*W + dx ; (dy, dx) = (R-1-r'-ph, S-1-s'-pw)
  };
  struct BState {};
  __device__ void a_init(AState& st, int m) const {
    if (m < M) {
      int c = mnv_fastdiv(m, g.d_RS);
      int rs = m - c * g.RS;
      int rp = mnv_fastdiv(rs, g.d_S);
      int sp = rs - rp * g.S;
      int dy = g.R - 1 - rp - g.ph, dx = g.S - 1 - sp - g.pw;
      st.off = c * g.HW + dy * g.W + dx;
      st.dyx = pack_yx(dy, dx);
    } else {
      st.off = 0;
      st.dyx = pack_yx(MNV_FAR, MNV_FAR);
    }
  }
  __device__ void b_init(BState&, int) const {}
  // A[m, kk..kk+3] = bottom[img, c, i*sv + dy, j*sh + dx] for kk = (img, i, j)
  __device__ void a_fetch(const AState& st, int, int k, float (&v)[4]) const {
    int img = mnv_fastdiv(k, g.d_HoWo);
    int pos = k - img * g.HoWo;
    int i = mnv_fastdiv(pos, g.d_Wo);
    int j = pos - i * g.Wo;
    const int dy = unpack_y(st.dyx), dx = unpack_x(st.dyx);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      int y = i * g.sv + dy, x = j * g.sh + dx;
      bool ok = (k + q < K) && (unsigned)y < (unsigned)g.H && (unsigned)x < (unsigned)g.W;
      v[q] = ok ? bottom[img * g.C * g.HW + st.off + i * g.sv * g.W + j * g.sh] : 0.f;
      if (++j == g.Wo) {
        j = 0;
        if (++i == g.Ho) {
          i = 0;
          ++img;
        }
      }
    }
  }
  // B[kk..kk+3, ko] = top_diff[img, ko, i, j]
  __device__ void b_fetch(const BState&, int n, int k, float (&v)[4]) const {
    int img = mnv_fastdiv(k, g.d_HoWo);
    int pos = k - img * g.HoWo;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      v[q] = (n < N && k + q < K) ? top_diff[((size_t)img * N + n) * g.HoWo + pos] : 0.f;
      if (++pos == g.HoWo) {
        pos = 0;
        ++img;
      }
    }
  }
  __device__ void c_store(int m, int n, float x) const { filter_diff[(size_t)n * M + m] = x; }
};

typedef MnvGemmTile<128, 128, 16, 2, 2> TileBig;
typedef MnvGemmTile<64, 64, 16, 2, 2> TileSmall;

int make_geom(ConvGeom* g, int N, int C, int K, int H, int W, int ph, int pw, int sv, int sh,
              int R, int S) {
  if (N <= 0 || C <= 0 || K <= 0 || H <= 0 || W <= 0 || ph < 0 || pw < 0 || sv <= 0 ||
      sh <= 0 || R <= 0 || S <= 0)
    return MNV_ERR_INVALID;
  int Ho = (H + 2 * ph - R) / sv + 1, Wo = (W + 2 * pw - S) / sh + 1;
  if (H + 2 * ph < R || W + 2 * pw < S || Ho <= 0 || Wo <= 0) return MNV_ERR_INVALID;
  // 16-bit packed coordinates and 32-bit element offsets
  if (H + ph + R >= 16000 || W + pw + S >= 16000) return MNV_ERR_INVALID;
  const long long lim = 0x7fffffffLL;
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

bool small_tiles(int m, int n) {
  long long big = (long long)((m + 127) / 128) * ((n + 127) / 128);
  return big < 128 || m <= 64 || n <= 64;
}

#define MNV_BWDF_MAX_SPLITS 256

int bwd_filter_splits(int m, int n, int k, size_t ws_floats) {
  bool small = small_tiles(m, n);
  int bm = small ? 64 : 128;
  long long tiles = (long long)((m + bm - 1) / bm) * ((n + bm - 1) / bm);
  int slabs = (k + 15) / 16;
  long long want = (1024 + tiles - 1) / tiles;
  if (want > MNV_BWDF_MAX_SPLITS) want = MNV_BWDF_MAX_SPLITS;
  if (want > slabs / 8) want = slabs / 8;
  size_t fit = ws_floats / ((size_t)m * n);
  if ((size_t)want > fit) want = (long long)fit;
  return want < 1 ? 1 : (int)want;
}

}  // namespace

extern "C" {

int mnv_conv_fwd(const float* bottom, const float* filter, const float* bias, float* top, int N,
                 int C, int K, int H, int W, int ph, int pw, int sv, int sh, int R, int S,
                 mnv_stream_t stream) {
  ConvGeom g;
  if (!bottom || !filter || !bias || !top) return MNV_ERR_INVALID;
  int rc = make_geom(&g, N, C, K, H, W, ph, pw, sv, sh, R, S);
  if (rc) return rc;
  int gm = N * g.HoWo, gn = K, gk = g.CRS;
  hipStream_t s = mnv_stream(stream);
  bool vecb = (gk % 4 == 0) && mnv_aligned16(filter);
  bool small = small_tiles(gm, gn);
  if (vecb) {
    ConvFwd<true> p{bottom, filter, bias, top, g, gm, gn, gk};
    return small ? mnv_gemm_launch<TileSmall>(p, 1, nullptr, s)
                 : mnv_gemm_launch<TileBig>(p, 1, nullptr, s);
  }
  ConvFwd<false> p{bottom, filter, bias, top, g, gm, gn, gk};
  return small ? mnv_gemm_launch<TileSmall>(p, 1, nullptr, s)
               : mnv_gemm_launch<TileBig>(p, 1, nullptr, s);
}

int mnv_conv_bwd_data(const float* top_diff, const float* filter, float* bottom_diff, int N,
                      int C, int K, int H, int W, int ph, int pw, int sv, int sh, int R, int S,
                      mnv_stream_t stream) {
  ConvGeom g;
  if (!top_diff || !filter || !bottom_diff) return MNV_ERR_INVALID;
  int rc = make_geom(&g, N, C, K, H, W, ph, pw, sv, sh, R, S);
  if (rc) return rc;
  int gm = N * g.HW, gn = C, gk = K * g.RS;
  ConvBwdData p{top_diff, filter, bottom_diff, g, gm, gn, gk};
  hipStream_t s = mnv_stream(stream);
  return small_tiles(gm, gn) ? mnv_gemm_launch<TileSmall>(p, 1, nullptr, s)
                             : mnv_gemm_launch<TileBig>(p, 1, nullptr, s);
}

size_t mnv_conv_bwd_filter_workspace_bytes(int N, int C, int K, int H, int W, int ph, int pw,
                                           int sv, int sh, int R, int S) {
  ConvGeom g;
  if (make_geom(&g, N, C, K, H, W, ph, pw, sv, sh, R, S)) return 0;
  int splits = bwd_filter_splits(g.CRS, K, N * g.HoWo, (size_t)-1);
  return splits > 1 ? (size_t)splits * g.CRS * K * sizeof(float) : 0;
}

int mnv_conv_bwd_filter(const float* bottom, const float* top_diff, float* filter_diff, int N,
                        int C, int K, int H, int W, int ph, int pw, int sv, int sh, int R, int S,
                        void* workspace, size_t workspace_bytes, mnv_stream_t stream) {
  ConvGeom g;
  if (!bottom || !top_diff || !filter_diff) return MNV_ERR_INVALID;
  int rc = make_geom(&g, N, C, K, H, W, ph, pw, sv, sh, R, S);
  if (rc) return rc;
  int gm = g.CRS, gn = K, gk = N * g.HoWo;
  ConvBwdFilter p{bottom, top_diff, filter_diff, g, gm, gn, gk};
  hipStream_t s = mnv_stream(stream);
  int splits = bwd_filter_splits(gm, gn, gk, workspace ? workspace_bytes / sizeof(float) : 0);
  return small_tiles(gm, gn) ? mnv_gemm_launch<TileSmall>(p, splits, workspace, s)
                             : mnv_gemm_launch<TileBig>(p, splits, workspace, s);
}

}  // extern "C"
