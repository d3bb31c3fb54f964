// fp32 MFMA GEMM core for gfx950, shared by SGEMM and the implicit-GEMM convolutions.
//
// Computes C[m,n] = sum_k A[m,k] * B[k,n] for one BM x BN tile per workgroup (and one
// k range per blockIdx.z when the k dimension is split).  The operands are described
// by a Problem policy: it knows how to fetch four values of A or B at once, either
// four consecutive m/n at one k ("x-fast", the natural direction of a column-major
// left operand or of an im2col gather) or four consecutive k at one m/n ("k-fast", a
// column-major right operand or a filter), and how to store an element of C.  So a
// convolution never materialises its im2col matrix: the gather happens on the way
// from HBM to LDS.
//
// Data path: HBM -> registers (policy fetch, issued one k-slab ahead) -> LDS, two
// slabs deep (double buffered, one barrier per slab) -> one fp32 value per lane per
// operand -> v_mfma_f32_32x32x2_f32.  Each wavefront owns a (TM*32) x (TN*32) block of
// accumulators.  The MFMA is issued with the operands swapped (B as the "A" input) so
// that the 64 lanes of an accumulator register hold 32 consecutive m: the C store of
// a column-major result is then 128 contiguous bytes per half wavefront.
//
// Roofline: fp32 MFMA, 2*M*N*K algorithmic flops; 256 flop/clk/CU.
#pragma once
#include <atomic>
#include <type_traits>

#include "mnv_common.h"

typedef float mnv_f16v __attribute__((ext_vector_type(16)));

#ifdef __HIPCC__
// BNU_ (default BN_): columns of the tile that are actually multiplied.  A tile fetches and
// stages BN columns but may compute only the first BNU of them (and tiles then advance by
// BNU), which lets a 96-wide output use three 32-column MFMA blocks instead of four.
template <int BM_, int BN_, int BK_, int WGM_, int WGN_, int PAD_ = 0, int BNU_ = BN_>
struct MnvGemmTile {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WGM = WGM_, WGN = WGN_, BNU = BNU_;
  static constexpr int NT = MNV_WAVE * WGM * WGN;
  static constexpr int WM = BM / WGM, WN = BNU / WGN;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int LDA = BM + PAD_, LDB = BN + PAD_;
  static constexpr int AV = BM * BK / (4 * NT);  // 4-vectors of A per thread per slab
  static constexpr int BV = BN * BK / (4 * NT);
  // LDS floats of one operand tile (one of two buffers).  An x-fast operand is stored
  // [k][x] (pitch LDA / LDB).  A k-fast operand is stored [x][k] with no padding, so that a
  // fetched 4-vector is one 16-byte LDS write and the MFMA side reads four k values per
  // 16-byte LDS read; the 16-byte chunks of row x are permuted by XOR with kswz(x), which
  // spreads both the writes (consecutive chunks of two rows per eight lanes) and the reads
  // (one chunk of eight consecutive rows) over all 32 banks.
  static constexpr int KCH = BK / 4;  // 16-byte chunks per row
  __host__ __device__ static constexpr int kswz(int x) { return (x / (32 / BK)) & (KCH - 1); }
  __host__ __device__ static constexpr int kaddr(int x, int chunk) {
    return x * BK + ((chunk ^ kswz(x)) << 2);
  }
  static constexpr int a_tile(bool kfast) { return kfast ? BM * BK : BK * LDA; }
  static constexpr int b_tile(bool kfast) { return kfast ? BN * BK : BK * LDB; }
  static constexpr size_t lds_bytes(bool a_kfast, bool b_kfast) {
    return (size_t)2 * (a_tile(a_kfast) + b_tile(b_kfast)) * sizeof(float);
  }
  // Wavefronts per SIMD the register allocation must allow: four 4-wavefront workgroups
  // per CU make 1024 resident tiles, which lets tile counts just under a multiple of
  // 1024 finish in whole rounds; two 8-wavefront workgroups are the same four wavefronts
  // per SIMD.
  static constexpr int MIN_WAVES = (NT == 256 && BM * BN <= 128 * 128 && BK <= 16) ? 4
                                   : (NT == 512 && BM * BN <= 256 * 128 && BK <= 16) ? 4 : 1;
  static_assert(WM % 32 == 0 && WN % 32 == 0 && BNU <= BN, "wave tile must be a multiple of 32x32");
  static_assert((BK == 8 || BK == 16 || BK == 32) && (BM * BK) % (4 * NT) == 0 &&
                    (BN * BK) % (4 * NT) == 0,
                "tile/thread mismatch");
};

// Per-thread position of its fetches inside an operand tile (BX x BK).
//  x-fast: vector p covers x = xg*4..+3 at k = kr + p*RP
//  k-fast: vector p covers k = kg*4..+3 at x = xc + p*CP
template <int BX, int BK, int NT, bool KFAST>
struct MnvFetchMap {
  static constexpr int GX = BX / 4, RP = NT / GX;  // x-fast
  static constexpr int GK = BK / 4, CP = NT / GK;  // k-fast
  static_assert(KFAST || (NT % GX == 0 && RP >= 1 && (BK % RP == 0 || RP > BK)), "x-fast map");
  static_assert(!KFAST || (NT % GK == 0 && BX % CP == 0), "k-fast map");
  __device__ static int x(int tid, int p) { return KFAST ? (tid / GK + p * CP) : (tid % GX) * 4; }
  __device__ static int k(int tid, int p) { return KFAST ? (tid % GK) * 4 : (tid / GX + p * RP); }
};

// Problem policy contract (all __device__ unless noted).  The k dimension is cut into
// slabs of BK and the slabs into "periods" of `spp` consecutive slabs: within a period
// every thread's byte offsets into A and B are constant and only a wavefront-uniform
// scalar offset advances, so a slab costs no address arithmetic at all (fp32 MFMA and
// VALU instructions do not overlap on gfx950: every VALU instruction in the main loop is
// matrix-pipe time lost).  Offsets are recomputed once per period.  A policy whose
// addressing has no such structure uses spp = 1.
//   static constexpr bool A_KFAST, B_KFAST;
//   static constexpr int A_NOFF, B_NOFF;      1: one 16-byte load per vector; 4: four 4-byte loads
//   int M, N, total_slabs, spp;               (host-set members)
//   struct Res;  void make_res(Res&) const;   buffer resources
//   struct AState / BState;                   per-thread, per-vector state set once
//   void a_init(const Res&, AState&, int m) const;    after block_init
//   void a_period(const AState&, unsigned (&off)[A_NOFF], int m, int kl, int period) const;
//        byte offsets of this vector's elements for slab 0 of `period`; kl = the vector's
//        first k index inside a slab; an element that must read as 0 gets MNV_OOB
//   void a_load(const Res&, const AState&, const unsigned (&off)[A_NOFF], int period, int s,
//               int kl, float (&v)[4]) const;
//        issues the loads of slab s of the period; the usual body is
//        mnv_fetch_vec(res.a, off, <uniform byte offset of the slab>, v)
//   (same for b with n)
//   size_t extra_lds_bytes() const;           (host) LDS the policy wants after the tiles
//   void block_init(Res&, float* extra_lds, int m0, int n0) const;   once per workgroup,
//        before the first load; a barrier follows it
//   void c_store(int m, int n, float v) const;   only called for m < M, n < N
//   optional, for a k-fast A whose k direction is contiguous in memory but whose rows are not
//   (the gathered operand of the filter gradient): static constexpr bool A_LANE_K = true;
//        The 16 k values of a slab then go to 16 consecutive lanes (a load instruction reads
//        64 contiguous bytes of each of four rows) and a thread holds one k of the rows
//        tid / 16 + 16 j.  a_init is called once, for row tid / 16, and
//   void a_load_lanek(const Res&, const AState&, int period, int s, int kl, float (&v)[AV][4]) const;
//        loads element j (row tid / 16 + 16 j, k = kl) into v[j / 4][j % 4]; a_period is unused
//   optional, for a right operand whose loads may fetch values that must read as 0 and that are
//   cheaper to clear once they have arrived: static constexpr bool B_STASH_FIX = true;
//   void b_stash_fix(int s, int kl, float (&v)[4]) const;   called on every vector of slab s of
//        its period right before the vector is written to LDS
//   optional, for an output whose m direction is contiguous in memory:
//   static constexpr bool C_STORE4 = true;
//   void c_store4(int m, int n, const float (&v)[4]) const;   the elements (m .. m + 3, n); m is a
//        multiple of 4 below M, the elements from M on are not to be stored
//        A launch without k ranges then passes every 32 x 32 block of accumulators through LDS
//        (a lane holds 4 consecutive n of one m, the store wants 4 consecutive m of one n) and
//        stores 16 bytes per lane, 512 contiguous bytes per column and instruction, instead of
//        4 bytes per lane: a quarter of the store instructions.  Taken for products of at most
//        MNV_STORE4_MAX_SLABS k-slabs.
//   optional, for a product whose left operand depends on the column tile (batched products
//   folded into the column index): static constexpr bool N_GROUPED = true;  int n_group;
//        Tiles are then dealt m-tile by m-tile within groups of n_group consecutive column
//        tiles (tiles_n is a multiple of n_group), so that the column tiles that read the
//        same A panel run next to each other; without it all m-tiles of one column tile come
//        first (the B panel is shared).  Not for stream-k launches.
//   optional, for a store that combines the product with a value read from memory:
//   static constexpr bool C_PRELOAD = true;
//   bool c_preload_on() const;                   uniform: whether this launch reads
//   float c_preload(int m, int n) const;         the value that goes with element (m,n)
//   void c_store_with(int m, int n, float v, float pre) const;
//        the kernel then reads the 16 values of a 32x32 block before it stores the block,
//        so the reads are in flight together instead of one ahead of each store
template <class P, class = void>
struct MnvALaneK {
  static constexpr bool value = false;
};
template <class P>
struct MnvALaneK<P, std::enable_if_t<P::A_LANE_K>> {
  static constexpr bool value = true;
};
template <class P, class = void>
struct MnvBStashFix {
  static constexpr bool value = false;
};
template <class P>
struct MnvBStashFix<P, std::enable_if_t<P::B_STASH_FIX>> {
  static constexpr bool value = true;
};
#define MNV_STORE4_MAX_SLABS 64
template <class P, class = void>
struct MnvCStore4 {
  static constexpr bool value = false;
};
template <class P>
struct MnvCStore4<P, std::enable_if_t<P::C_STORE4>> {
  static constexpr bool value = true;
};
template <class P, class = void>
struct MnvNGrouped {
  static constexpr bool value = false;
};
template <class P>
struct MnvNGrouped<P, std::enable_if_t<P::N_GROUPED>> {
  static constexpr bool value = true;
};
template <class P, class = void>
struct MnvCPreload {
  static constexpr bool value = false;
};
template <class P>
struct MnvCPreload<P, std::enable_if_t<P::C_PRELOAD>> {
  static constexpr bool value = true;
};
template <int NOFF>
__device__ __forceinline__ void mnv_fetch_vec(mnv_rsrc r, const unsigned (&off)[NOFF],
                                              unsigned soff, float (&v)[4]) {
  if (NOFF == 1) {
    mnv_f4 t = __builtin_bit_cast(
        mnv_f4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)off[0], (int)soff, 0));
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  } else {
#pragma unroll
    for (int q = 0; q < 4; ++q)
      v[q] = __builtin_bit_cast(
          float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)off[q % NOFF], (int)soff, 0));
  }
}

// Workgroups are dealt round-robin to the 8 XCDs; the tile index is remapped so that each XCD
// (one L2) works on a contiguous run of tiles that share B panels.
__device__ __forceinline__ int mnv_tile_remap(int t, int total) {
  const int per_xcd = total / 8;
  return t < per_xcd * 8 ? (t % 8) * per_xcd + t / 8 : t;
}

// Tile coordinates of the (remapped) tile index b.
template <class P>
__device__ __forceinline__ void mnv_tile_coords(const P& prob, int b, int tiles_m, int& tile_m,
                                                int& tile_n) {
  if constexpr (MnvNGrouped<P>::value) {
    const int per = tiles_m * prob.n_group;
    const int grp = b / per, r = b - grp * per;
    tile_m = r / prob.n_group;
    tile_n = grp * prob.n_group + (r - tile_m * prob.n_group);
  } else {
    tile_m = b % tiles_m;
    tile_n = b / tiles_m;
  }
}

// Tail: tiles are whole units of work, so when their number is not a multiple of the CU
// count the CUs that receive one tile more than the others set the duration (676 tiles on 256
// CUs: three on some, 2.64 on average).  The tiles past the last multiple (`tail_begin`
// on, in dispatch order) are therefore cut into `tail_z` k ranges, one workgroup each: small
// units that are dispatched last and fill the CUs evenly.  Their partial tiles go to the
// workspace, tile by tile, and mnv_gemm_tail_reduce_kernel adds them in range order.
//
// G > 1: the workgroup is G groups of T::NT threads that work on the same output tile.
// Each group has its own pair of LDS buffers and multiplies its own quarter of the
// workgroup's k range; at the end the groups' accumulators are added through LDS in a fixed
// order ((g0 + g2) + (g1 + g3)) and group 0 stores.  For a product with few output tiles and
// a long k this keeps 16 wavefronts per CU busy with a quarter of the partial results (and of
// the reduction kernel's reads) that as many separate workgroups would write to memory.
//
// SK ("stream-k"): the launch has exactly as many workgroups as the chip holds at once (W) and
// every one of them multiplies the same number of k-slabs, U / W of the U = tiles x slabs units
// of the whole product.  With T tiles, Z = W / T of every tile's k ranges are "aligned": range
// z of every tile covers the same slabs [z CH, (z + 1) CH), CH = U / W, one workgroup each,
// and the workgroups of one range sit side by side on one XCD (the launch index is remapped
// as for the tiles of a plain launch) -- they start together, run at the same pace and so
// read the same operand panels at the same time, out of that XCD's L2.  What the aligned
// ranges leave of every tile, the slabs from Z CH on, is laid end to end (tile-major) and
// dealt in equal contiguous shares to the R = W - T Z workgroups that remain (none when T
// divides W: the Z ranges then cut the tile evenly); such a share crosses tile boundaries and
// is worked off segment by segment.  Every aligned range leaves its partial tile in slot
// z T + tile of the workspace, every segment of remaining workgroup r in slot T Z + r + tile (r
// and tile never decrease from one segment to the next and one of them grows, so the slots
// are distinct, W + T at most), and mnv_gemm_streamk_reduce_kernel adds a tile's partial tiles
// in k order: deterministic.  With whole k ranges per workgroup (blockIdx.z) the chip works in
// rounds of equal workgroups, and a count of workgroups that is not a multiple of what the
// chip holds leaves part of it idle for a whole round (54 tiles x 28 ranges = 1512 workgroups
// on 1024 slots: the second round runs half empty).  Equal contiguous shares of the units
// laid end to end without aligned ranges balance as well but no two workgroups ever read the
// same panel at the same time: measured on the padded convolutions' filter gradients of the
// AlexNet shape, 5.3 GB of L2 fills per launch for 3.9 GB of operand reads, and 3% slower
// than whole ranges of 729 to 760 workgroups on 768 slots.
//
// PF: slabs the loads run ahead of the multiplies.  1: the loads of slab i + 1 are issued at
// the head of slab i and written to LDS at its end, through one set of staging registers
// (the kernel then fits 128 registers: four workgroups per CU).  2: a second set of staging
// registers lets the loads of slab i + 2 start at the head of slab i, so that a trip to
// memory may take two slab times instead of one; 24 more registers, three workgroups per CU.
// Partial tiles (the k ranges of a cut tail, the ranges and segments of a stream-k launch) are
// private to this file, so they are kept in the order the accumulators have in registers:
// 16-byte group q of thread t, i.e. the accumulators 4 g .. 4 g + 3 of the thread's block (i, j)
// with q = (i TN + j) 4 + g, sits at float (q NT + t) 4.  A thread then writes its tile in
// TM x TN x 4 fully coalesced 16-byte stores instead of 16 times as many 4-byte ones.  The
// four floats of a group are four consecutive n of one m:
template <class T>
__device__ __forceinline__ void mnv_partial_group_mn(int group, int& m, int& n) {
  const int q = group / T::NT, t = group - q * T::NT;
  const int wave = t / MNV_WAVE, lane = t % MNV_WAVE;
  const int i = q / (T::TN * 4), j = (q / 4) % T::TN, g = q % 4;
  m = (wave % T::WGM) * T::WM + i * 32 + lane % 32;
  n = (wave / T::WGM) * T::WN + j * 32 + (lane / 32) * 4 + 8 * g;
}
template <class T, class P, int G = 1, bool SK = false, int PF = 1>
__global__ __launch_bounds__(T::NT * G, PF == 2 && T::MIN_WAVES == 4 ? 3 : T::MIN_WAVES) void mnv_gemm_kernel(
    P prob, int tiles_m, int tiles_n, int slabs_per_split, float* __restrict__ partial,
    int tail_begin, int tail_z) {
  static_assert(!SK || G == 1, "stream-k shares are per workgroup");
  static_assert(PF == 1 || (PF == 2 && G == 1), "one or two slabs ahead");
  extern __shared__ float mnv_gemm_lds[];
  constexpr int ATILE = T::a_tile(P::A_KFAST), BTILE = T::b_tile(P::B_KFAST);
  constexpr int GROUP_FLOATS = 2 * (ATILE + BTILE);
  static_assert(G == 1 || G == 4, "one group, or four that are added pairwise");
  const int tid = G > 1 ? (int)(threadIdx.x % T::NT) : (int)threadIdx.x;
  const int grp = G > 1 ? __builtin_amdgcn_readfirstlane((int)(threadIdx.x / T::NT)) : 0;
  float* As = mnv_gemm_lds + grp * GROUP_FLOATS;  // two buffers of ATILE floats
  float* Bs = As + 2 * ATILE;                     // two buffers of BTILE floats
  typedef MnvFetchMap<T::BM, T::BK, T::NT, P::A_KFAST> MapA;
  typedef MnvFetchMap<T::BN, T::BK, T::NT, P::B_KFAST> MapB;

  // SK: slabs_per_split = CH, tail_begin = Z.  sk_p: this workgroup's place in the plan (an
  // aligned range below T Z, else a remaining workgroup); sk_u, sk_end: the remaining
  // workgroup's units, counted over the slabs the aligned ranges leave, that are still to do.
  long long sk_u = 0, sk_end = 0;
  int sk_p = 0, sk_aligned = 0, sk_rest = 0;  // sk_rest: slabs per tile past the aligned ranges
  if constexpr (SK) {
    const int tiles = tiles_m * tiles_n, aligned = tiles * tail_begin;
    const int rem = (int)gridDim.x - aligned;
    sk_p = mnv_tile_remap((int)blockIdx.x, (int)gridDim.x);
    sk_aligned = sk_p < aligned;
    sk_rest = prob.total_slabs - tail_begin * slabs_per_split;
    if (!sk_aligned) {
      const long long units = (long long)sk_rest * tiles;
      sk_u = units * (sk_p - aligned) / rem;
      sk_end = units * (sk_p - aligned + 1) / rem;
      if (sk_u >= sk_end) return;
    }
  }
  for (;;) {  // SK: one pass per segment; otherwise a single pass that ends in a return
  int vb = blockIdx.x, tail_part = -1;
  if (!SK && G == 1 && tail_z > 1 && vb >= tail_begin) {
    const int i = vb - tail_begin, tl = i / tail_z;
    tail_part = i - tl * tail_z;
    vb = tail_begin + tl;
  }
  int sk_z = 0;
  if constexpr (SK) {
    if (sk_aligned) {
      sk_z = sk_p / (tiles_m * tiles_n);
      vb = sk_p - sk_z * (tiles_m * tiles_n);
    } else {
      vb = (int)(sk_u / sk_rest);
    }
  }
  const int b = SK ? vb : mnv_tile_remap(vb, tiles_m * tiles_n);
  int tile_m, tile_n;
  if constexpr (SK) {
    tile_m = b % tiles_m;
    tile_n = b / tiles_m;
  } else {
    mnv_tile_coords(prob, b, tiles_m, tile_m, tile_n);
  }
  const int m0 = tile_m * T::BM, n0 = tile_n * T::BNU;

  int slab_begin = blockIdx.z * slabs_per_split;
  int slab_end = slab_begin + slabs_per_split;
  if (slab_end > prob.total_slabs) slab_end = prob.total_slabs;
  if constexpr (SK) {
    if (sk_aligned) {
      if ((int)gridDim.x == tiles_m * tiles_n * tail_begin) {  // no remaining workgroups: even cuts
        slab_begin = (int)((long long)prob.total_slabs * sk_z / tail_begin);
        slab_end = (int)((long long)prob.total_slabs * (sk_z + 1) / tail_begin);
      } else {
        slab_begin = sk_z * slabs_per_split;
        slab_end = slab_begin + slabs_per_split;
      }
    } else {
      slab_begin = prob.total_slabs - sk_rest + (int)(sk_u - (long long)vb * sk_rest);
      const long long left = sk_end - sk_u;
      slab_end = left < prob.total_slabs - slab_begin ? slab_begin + (int)left : prob.total_slabs;
    }
  }
  // slabs every group steps through (the same count in all of them: the steps hold
  // workgroup barriers); a group whose quarter is shorter multiplies only its own slabs
  if (G == 1 && tail_part >= 0) {
    const int per = (prob.total_slabs + tail_z - 1) / tail_z;
    slab_begin = tail_part * per;
    slab_end = slab_begin + per < prob.total_slabs ? slab_begin + per : prob.total_slabs;
    if (slab_begin > slab_end) slab_begin = slab_end;
  }
  int trips = slab_end - slab_begin;
  if (G > 1) {
    trips = (trips + G - 1) / G;
    slab_begin += grp * trips;
    if (slab_begin > slab_end) slab_begin = slab_end;
    if (slab_end > slab_begin + trips) slab_end = slab_begin + trips;
  }

  typename P::Res res;
  prob.make_res(res);
  prob.block_init(res, mnv_gemm_lds + G * GROUP_FLOATS, m0, n0);
  typename P::AState ast[T::AV];
  typename P::BState bst[T::BV];
  unsigned aoff[T::AV][P::A_NOFF], boff[T::BV][P::B_NOFF];
  constexpr bool LK = MnvALaneK<P>::value;
  static_assert(!LK || (P::A_KFAST && T::BK == 16 && T::NT == 256), "lane-per-k fetch: 16 x 16 threads");
  if constexpr (LK) {
    prob.a_init(res, ast[0], m0 + tid / 16);
  } else {
#pragma unroll
    for (int p = 0; p < T::AV; ++p) prob.a_init(res, ast[p], m0 + MapA::x(tid, p));
  }
#pragma unroll
  for (int p = 0; p < T::BV; ++p) prob.b_init(res, bst[p], n0 + MapB::x(tid, p));

  float ra[PF][T::AV][4], rb[PF][T::BV][4];  // staging set of slab j: j % PF

  auto new_period = [&](int period) {
    if constexpr (!LK) {
#pragma unroll
      for (int p = 0; p < T::AV; ++p)
        prob.a_period(ast[p], aoff[p], m0 + MapA::x(tid, p), MapA::k(tid, p), period);
    }
#pragma unroll
    for (int p = 0; p < T::BV; ++p)
      prob.b_period(bst[p], boff[p], n0 + MapB::x(tid, p), MapB::k(tid, p), period);
  };
  int s_of_set[PF] = {};  // slab (inside its period) that each staging set holds
  auto fetch = [&](int period, int s, auto SET) {
    constexpr int set = decltype(SET)::value;
    s_of_set[set] = s;
    if constexpr (LK) {
      prob.a_load_lanek(res, ast[0], period, s, tid % 16, ra[set]);
    } else {
#pragma unroll
      for (int p = 0; p < T::AV; ++p)
        prob.a_load(res, ast[p], aoff[p], period, s, MapA::k(tid, p), ra[set][p]);
    }
#pragma unroll
    for (int p = 0; p < T::BV; ++p)
      prob.b_load(res, bst[p], boff[p], period, s, MapB::k(tid, p), rb[set][p]);
  };
  auto stash = [&](int buf, auto SET) {
    constexpr int set = decltype(SET)::value;
    float* a = As + buf * ATILE;
    float* bb = Bs + buf * BTILE;
    if constexpr (MnvBStashFix<P>::value) {
#pragma unroll
      for (int p = 0; p < T::BV; ++p) prob.b_stash_fix(s_of_set[set], MapB::k(tid, p), rb[set][p]);
    }
    if constexpr (LK) {  // element j: row tid / 16 + 16 j, k = tid % 16
#pragma unroll
      for (int j = 0; j < T::AV * 4; ++j)
        a[T::kaddr(tid / 16 + 16 * j, (tid % 16) >> 2) + (tid & 3)] = ra[set][j / 4][j % 4];
    } else {
#pragma unroll
      for (int p = 0; p < T::AV; ++p) {
        const int x = MapA::x(tid, p), k = MapA::k(tid, p);
        mnv_f4 v = {ra[set][p][0], ra[set][p][1], ra[set][p][2], ra[set][p][3]};
        *reinterpret_cast<mnv_f4*>(a + (P::A_KFAST ? T::kaddr(x, k >> 2) : k * T::LDA + x)) = v;
      }
    }
#pragma unroll
    for (int p = 0; p < T::BV; ++p) {
      const int x = MapB::x(tid, p), k = MapB::k(tid, p);
      mnv_f4 v = {rb[set][p][0], rb[set][p][1], rb[set][p][2], rb[set][p][3]};
      *reinterpret_cast<mnv_f4*>(bb + (P::B_KFAST ? T::kaddr(x, k >> 2) : k * T::LDB + x)) = v;
    }
  };

  mnv_f16v acc[T::TM][T::TN];
#pragma unroll
  for (int i = 0; i < T::TM; ++i)
#pragma unroll
    for (int j = 0; j < T::TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int wave = tid / MNV_WAVE, lane = tid % MNV_WAVE;
  const int wm = (wave % T::WGM) * T::WM, wn = (wave / T::WGM) * T::WN;
  const int lm = lane % 32, lk = lane / 32;

  // (period, s) of the slab whose loads are issued next
  int period = slab_begin / prob.spp, s = slab_begin - period * prob.spp;
  __syncthreads();  // block_init may have written LDS
  typedef std::integral_constant<int, 0> Set0;
  typedef std::integral_constant<int, PF - 1> Set1;
  if (slab_begin < slab_end) {
    new_period(period);
    fetch(period, s, Set0{});
    if constexpr (PF == 2) {
      if (++s == prob.spp) {
        s = 0;
        new_period(++period);
      }
      fetch(period, s, Set1{});
    }
    stash(0, Set0{});
  }
  __syncthreads();

  // One slab out of LDS buffer BUF.  The buffer is a compile-time constant (the loop below
  // is unrolled by two) so that the LDS addresses of both buffers are one register plus an
  // immediate: selecting the buffer at run time cost seven address instructions per slab,
  // and every vector instruction in this loop is time the matrix pipe stands still.
  auto step = [&](auto BUF, bool active) {
    constexpr int buf = decltype(BUF)::value;
    // Loads of the next slab are in flight while this one is multiplied.  Past the end of
    // the k range the loads run past the tensors and read as 0 (or fetch a slab of the
    // next split, which is never multiplied).
    if (++s == prob.spp) {
      s = 0;
      new_period(++period);
    }
    fetch(period, s, std::integral_constant<int, PF == 2 ? buf : 0>{});
    // One slab ahead, keep the loads up here: left alone, the scheduler sinks them below most
    // of the multiplies to shorten register lifetimes, and each wavefront then waits out the
    // full memory latency once per slab.  Two slabs ahead that is exactly what is wanted: the
    // loads have a whole slab of slack, and issued in the shadow of the multiplies they cost
    // the wavefront no issue slots at the head of the slab, where its four operand reads and
    // the first multiply wait (filter gradients of the AlexNet shape: 1.014 -> 0.987 ms).
    if (PF == 1) __builtin_amdgcn_sched_barrier(0);
    // A round multiplies 8 k values: MFMA step t pairs k = 8h + t (lanes 0..31) with
    // k = 8h + 4 + t (lanes 32..63), so a lane's four steps use four consecutive k.
    const float* a = As + buf * ATILE;
    const float* bb = Bs + buf * BTILE;
    if (G == 1 || active) {
#pragma unroll
    for (int h = 0; h < T::BK / 8; ++h) {
      float av[T::TM][4], bv[T::TN][4];
      const int kq = 8 * h + 4 * lk;
#pragma unroll
      for (int i = 0; i < T::TM; ++i) {
        const int x = wm + i * 32 + lm;
        if (P::A_KFAST) {
          mnv_f4 v = *reinterpret_cast<const mnv_f4*>(a + T::kaddr(x, kq >> 2));
          av[i][0] = v.x; av[i][1] = v.y; av[i][2] = v.z; av[i][3] = v.w;
        } else {
#pragma unroll
          for (int t = 0; t < 4; ++t) av[i][t] = a[(kq + t) * T::LDA + x];
        }
      }
#pragma unroll
      for (int j = 0; j < T::TN; ++j) {
        const int x = wn + j * 32 + lm;
        if (P::B_KFAST) {
          mnv_f4 v = *reinterpret_cast<const mnv_f4*>(bb + T::kaddr(x, kq >> 2));
          bv[j][0] = v.x; bv[j][1] = v.y; bv[j][2] = v.z; bv[j][3] = v.w;
        } else {
#pragma unroll
          for (int t = 0; t < 4; ++t) bv[j][t] = bb[(kq + t) * T::LDB + x];
        }
      }
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < T::TM; ++i)
#pragma unroll
          for (int j = 0; j < T::TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[j][t], av[i][t], acc[i][j], 0, 0, 0);
    }
    }
    stash(buf ^ 1, std::integral_constant<int, PF == 2 ? (buf ^ 1) : 0>{});
    __syncthreads();
  };
  int slab = slab_begin;
  const int loop_end = slab_begin + trips;
  for (; slab + 1 < loop_end; slab += 2) {
    step(std::integral_constant<int, 0>{}, slab < slab_end);
    step(std::integral_constant<int, 1>{}, slab + 1 < slab_end);
  }
  if (slab < loop_end) step(std::integral_constant<int, 0>{}, slab < slab_end);

  if constexpr (G > 1) {
    // Every wavefront has passed the last step's barrier: the tile buffers are free and
    // hold two groups' accumulators at a time, register by register (consecutive lanes at
    // consecutive addresses).
    constexpr int PART = T::NT * T::TM * T::TN * 16;
    static_assert(2 * PART <= G * GROUP_FLOATS, "two partial tiles must fit the tile buffers");
    float* red = mnv_gemm_lds;
    auto put = [&](int region) {
#pragma unroll
      for (int i = 0; i < T::TM; ++i)
#pragma unroll
        for (int j = 0; j < T::TN; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            red[region * PART + ((i * T::TN + j) * 16 + r) * T::NT + tid] = acc[i][j][r];
    };
    auto add = [&](int region) {
#pragma unroll
      for (int i = 0; i < T::TM; ++i)
#pragma unroll
        for (int j = 0; j < T::TN; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            acc[i][j][r] += red[region * PART + ((i * T::TN + j) * 16 + r) * T::NT + tid];
    };
    if (grp >= 2) put(grp - 2);
    __syncthreads();
    if (grp < 2) add(grp);
    __syncthreads();
    if (grp == 1) put(0);
    __syncthreads();
    if (grp != 0) return;
    add(0);
  }

  // Accumulator register r of lane (lm, lk) holds C[m = lm, n = lk*4 + r%4 + 8*(r/4)]
  // of its 32x32 block.
  if constexpr (SK) {  // a range or a segment: the whole tile, in register order, into its slot
    // The empty asm keeps the store addresses from being computed once before the segment
    // loop (they do not change from segment to segment): 64 registers held across the main
    // loop would spill.
    int at = tid * 4;
    asm volatile("" : "+v"(at));
    float* pt = partial + (size_t)(sk_aligned ? sk_p : sk_p + vb) * (T::BM * T::BNU) + at;
#pragma unroll
    for (int i = 0; i < T::TM; ++i)
#pragma unroll
      for (int j = 0; j < T::TN; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const mnv_f4 v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
          *reinterpret_cast<mnv_f4*>(pt + ((i * T::TN + j) * 4 + g) * (T::NT * 4)) = v;
        }
    if (sk_aligned) return;
    sk_u += slab_end - slab_begin;
    if (sk_u >= sk_end) return;
    // every wavefront is past the last slab's barrier: the tile buffers and the policy's
    // LDS are free for the next segment
    continue;
  }
  if (G == 1 && tail_part >= 0) {  // a k range of a tail tile: the whole tile, in register order
    float* pt = partial + ((size_t)(vb - tail_begin) * tail_z + tail_part) * (T::BM * T::BNU) + tid * 4;
#pragma unroll
    for (int i = 0; i < T::TM; ++i)
#pragma unroll
      for (int j = 0; j < T::TN; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const mnv_f4 v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
          *reinterpret_cast<mnv_f4*>(pt + ((i * T::TN + j) * 4 + g) * (T::NT * 4)) = v;
        }
    return;
  }
  const bool split = gridDim.z > 1;
  float* part = split ? partial + (size_t)blockIdx.z * prob.M * prob.N : nullptr;
  // rows x columns of one pass through LDS: one 32 x 32 block of every wavefront
  constexpr int SROWS = T::WGM * 32, SCOLS = T::WGN * 32, SPITCH = SROWS + 4;
  if constexpr (MnvCStore4<P>::value && G == 1 && SCOLS * SPITCH <= GROUP_FLOATS &&
                (SCOLS * (SROWS / 4)) % T::NT == 0) {
    // Worth it where the stores are a large part of a tile's time, i.e. for a short k
    // (measured: conv1 forward of the AlexNet shape, 23 slabs, 0.526 -> 0.482 ms; 4096 x 9216
    // x 256, 16 slabs, 0.177 -> 0.161 ms; with 144-216 slabs the two extra barriers per block
    // cost the data gradients 2% and gain the forward kernels nothing)
    bool direct = !split && prob.total_slabs <= MNV_STORE4_MAX_SLABS;
    if constexpr (MnvCPreload<P>::value) direct = direct && !prob.c_preload_on();
    if (direct) {
      // every wavefront is past the last slab's barrier: the tile buffers are free
      float* stage = mnv_gemm_lds;
      const int srow = (wave % T::WGM) * 32 + lm, scol = (wave / T::WGM) * 32 + lk * 4;
      constexpr int QPC = SROWS / 4;                    // 16-byte groups per column
      constexpr int PER = SCOLS * QPC / T::NT;          // groups per thread and pass
#pragma unroll
      for (int i = 0; i < T::TM; ++i)
#pragma unroll
        for (int j = 0; j < T::TN; ++j) {
#pragma unroll
          for (int r = 0; r < 16; ++r)
            stage[(scol + (r & 3) + 8 * (r >> 2)) * SPITCH + srow] = acc[i][j][r];
          __syncthreads();
#pragma unroll
          for (int q = 0; q < PER; ++q) {
            const int idx = q * T::NT + tid, col = idx / QPC, row = (idx - col * QPC) * 4;
            const mnv_f4 v = *reinterpret_cast<const mnv_f4*>(stage + col * SPITCH + row);
            const int m = m0 + (row / 32) * T::WM + i * 32 + row % 32;
            const int n = n0 + (col / 32) * T::WN + j * 32 + col % 32;
            if (m < prob.M && n < prob.N) {
              const float x[4] = {v.x, v.y, v.z, v.w};
              prob.c_store4(m, n, x);
            }
          }
          __syncthreads();
        }
      return;
    }
  }
  if constexpr (MnvCPreload<P>::value) {
    if (!split && prob.c_preload_on()) {
#pragma unroll
      for (int i = 0; i < T::TM; ++i) {
        const int m = m0 + wm + i * 32 + lm;
        if (m >= prob.M) continue;
#pragma unroll
        for (int j = 0; j < T::TN; ++j) {
          float pre[16];
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int n = n0 + wn + j * 32 + lk * 4 + (r & 3) + 8 * (r >> 2);
            pre[r] = n < prob.N ? prob.c_preload(m, n) : 0.f;
          }
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int n = n0 + wn + j * 32 + lk * 4 + (r & 3) + 8 * (r >> 2);
            if (n < prob.N) prob.c_store_with(m, n, acc[i][j][r], pre[r]);
          }
        }
      }
      return;
    }
  }
#pragma unroll
  for (int i = 0; i < T::TM; ++i) {
    const int m = m0 + wm + i * 32 + lm;
    if (m >= prob.M) continue;
#pragma unroll
    for (int j = 0; j < T::TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int n = n0 + wn + j * 32 + lk * 4 + (r & 3) + 8 * (r >> 2);
        if (n < prob.N) {
          if (split) part[(size_t)n * prob.M + m] = acc[i][j][r];
          else prob.c_store(m, n, acc[i][j][r]);
        }
      }
  }
  return;
  }  // for (;;)
}

// Sums the per-split partial results in a fixed order (deterministic) and hands each
// element to the policy's store.  ZL threads share one output element: thread z of them
// adds the partial results z, z + ZL, z + 2 ZL, ... and the ZL sums are added in order
// through LDS.  A small output with many k ranges (the filter gradient of a narrow
// convolution: a few hundred elements, hundreds of ranges) would otherwise leave the chip
// to a few hundred threads that each walk the whole list.
template <class P, int ZL>
__global__ __launch_bounds__(256) void mnv_gemm_splitk_reduce_kernel(P prob,
                                                                    const float* __restrict__ partial,
                                                                    int splits) {
  constexpr int QL = 256 / ZL;  // output elements per workgroup pass
  __shared__ float red[ZL > 1 ? 256 : 1];
  const size_t mn = (size_t)prob.M * prob.N;
  const int tq = threadIdx.x % QL, tz = threadIdx.x / QL;
  for (size_t q0 = (size_t)blockIdx.x * QL; q0 < mn; q0 += (size_t)gridDim.x * QL) {
    const size_t q = q0 + tq;
    float s = 0.f;
    if (q < mn) {
      const float* p = partial + q + (size_t)tz * mn;
      const size_t step = (size_t)ZL * mn;
      int z = tz;
      float v0, v1, v2, v3;
      for (; z + 3 * ZL < splits; z += 4 * ZL, p += 4 * step) {
        v0 = p[0]; v1 = p[step]; v2 = p[2 * step]; v3 = p[3 * step];
        s += v0; s += v1; s += v2; s += v3;
      }
      for (; z < splits; z += ZL, p += step) s += *p;
    }
    if (ZL == 1) {
      if (q < mn) prob.c_store((int)(q % prob.M), (int)(q / prob.M), s);
    } else {
      __syncthreads();  // the previous pass has read its sums
      red[threadIdx.x] = s;
      __syncthreads();
      if (tz == 0 && q < mn) {
        float t = red[tq];
#pragma unroll
        for (int z = 1; z < ZL; ++z) t += red[z * QL + tq];
        prob.c_store((int)(q % prob.M), (int)(q / prob.M), t);
      }
    }
  }
}

template <class P, int ZL>
static int mnv_gemm_splitk_reduce_launch(const P& prob, const float* partial, int splits,
                                         hipStream_t s) {
  const size_t mn = (size_t)prob.M * prob.N;
  size_t blocks = mnv_ceil_div(mn, 256 / ZL);
  if (blocks > MNV_MAX_STREAM_BLOCKS) blocks = MNV_MAX_STREAM_BLOCKS;
  hipLaunchKernelGGL((mnv_gemm_splitk_reduce_kernel<P, ZL>), dim3((unsigned)blocks), dim3(256), 0,
                     s, prob, partial, splits);
  return MNV_LAUNCH_STATUS();
}

// Adds the k ranges of the tail tiles (see mnv_gemm_kernel) in range order and hands every
// element to the policy's store.  One thread per 16-byte group of the partial tiles (register
// order, see mnv_partial_group_mn): four consecutive columns of one row.
template <class T, class P>
__global__ __launch_bounds__(256) void mnv_gemm_tail_reduce_kernel(P prob,
                                                                   const float* __restrict__ partial,
                                                                   int tiles_m, int tiles_n,
                                                                   int tail_begin, int tail_z) {
  constexpr int TILE = T::BM * T::BNU;
  const int b = mnv_tile_remap(tail_begin + (int)blockIdx.y, tiles_m * tiles_n);
  int tile_m, tile_n;
  mnv_tile_coords(prob, b, tiles_m, tile_m, tile_n);
  const int m0 = tile_m * T::BM, n0 = tile_n * T::BNU;
  const float* p = partial + (size_t)blockIdx.y * tail_z * TILE;
  for (int e = (blockIdx.x * 256 + threadIdx.x) * 4; e < TILE; e += gridDim.x * 256 * 4) {
    mnv_f4 s = *reinterpret_cast<const mnv_f4*>(p + e);
    for (int z = 1; z < tail_z; ++z) {
      const mnv_f4 v = *reinterpret_cast<const mnv_f4*>(p + (size_t)z * TILE + e);
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    int m, n;
    mnv_partial_group_mn<T>(e / 4, m, n);
    m += m0;
    n += n0;
    if (m < prob.M) {
      if (n + 0 < prob.N) prob.c_store(m, n + 0, s.x);
      if (n + 1 < prob.N) prob.c_store(m, n + 1, s.y);
      if (n + 2 < prob.N) prob.c_store(m, n + 2, s.z);
      if (n + 3 < prob.N) prob.c_store(m, n + 3, s.w);
    }
  }
}

// Adds the partial tiles of every tile of a stream-k launch (see mnv_gemm_kernel) in k order and
// hands each element to the policy's store.  Tile t has the `aligned` ranges' partial tiles in
// the slots z T + t and, when the launch had R = W - T aligned remaining workgroups, the
// segments of those that met the tile: remaining workgroup r covered the units [U r / R,
// U (r + 1) / R) of the U = T `rest` slabs the aligned ranges left, tile t is the units [t rest,
// (t + 1) rest), and the segment sits in slot T aligned + r + t.  A thread owns one 16-byte
// group of the tile (register order, see mnv_partial_group_mn); ZL threads share it: thread z adds the partial tiles z,
// z + ZL, ... in order, and the ZL sums are added in order through LDS.  An output of few
// tiles has hundreds of partial tiles per tile (three tiles on 768 workgroups: 256 each),
// which one thread per element walked in 52 us; sixteen walk them in a quarter of that.
template <class T, class P, int ZL>
__global__ __launch_bounds__(256) void mnv_gemm_streamk_reduce_kernel(P prob,
                                                                      const float* __restrict__ partial,
                                                                      int tiles_m, int tiles_n,
                                                                      int workgroups, int aligned,
                                                                      int rest) {
  constexpr int TILE = T::BM * T::BNU;
  constexpr int QL = 256 / ZL;  // 4-vectors of a tile per workgroup
  __shared__ mnv_f4 red[ZL > 1 ? 256 : 1];
  const int t = blockIdx.y, tiles = tiles_m * tiles_n;
  const long long R = workgroups - (long long)tiles * aligned;
  int seg_first = 0, segs = 0;  // remaining workgroups that met the tile
  if (R > 0) {
    const long long S = rest, U = S * tiles;
    const long long first = t * S, last = first + S;
    long long w0 = first * R / U;                  // U w0 / R <= first
    while (U * (w0 + 1) / R <= first) ++w0;        // the share that holds the tile's first unit
    long long w1 = (last * R + U - 1) / U;         // the first share that begins at or past the
    while (w1 > w0 + 1 && U * (w1 - 1) / R >= last) --w1;  // tile's end (a step or two of rounding,
    while (w1 < R && U * w1 / R < last) ++w1;              // not a walk over the shares)
    seg_first = (int)w0;
    segs = (int)(w1 - w0);
  }
  const int m0 = (t % tiles_m) * T::BM, n0 = (t / tiles_m) * T::BNU;
  const int count = aligned + segs;
  // partial tile i of the tile, in k order
  const float* p = partial + (size_t)t * TILE;
  const float* pseg = partial + ((size_t)tiles * aligned + seg_first + t) * TILE;
  auto part = [&](int i) -> const float* {
    return i < aligned ? p + (size_t)i * tiles * TILE : pseg + (size_t)(i - aligned) * TILE;
  };
  const int tq = threadIdx.x % QL, tz = threadIdx.x / QL;
  static_assert(TILE % (4 * QL) == 0, "whole passes");
  for (int e = (blockIdx.x * QL + tq) * 4; e < TILE; e += gridDim.x * QL * 4) {
    mnv_f4 s = {0.f, 0.f, 0.f, 0.f};
    int z = tz;
    if (z < count) {
      s = *reinterpret_cast<const mnv_f4*>(part(z) + e);
      z += ZL;
    }
    for (; z + 3 * ZL < count; z += 4 * ZL) {
      const mnv_f4 v0 = *reinterpret_cast<const mnv_f4*>(part(z) + e);
      const mnv_f4 v1 = *reinterpret_cast<const mnv_f4*>(part(z + ZL) + e);
      const mnv_f4 v2 = *reinterpret_cast<const mnv_f4*>(part(z + 2 * ZL) + e);
      const mnv_f4 v3 = *reinterpret_cast<const mnv_f4*>(part(z + 3 * ZL) + e);
      s.x += v0.x; s.y += v0.y; s.z += v0.z; s.w += v0.w;
      s.x += v1.x; s.y += v1.y; s.z += v1.z; s.w += v1.w;
      s.x += v2.x; s.y += v2.y; s.z += v2.z; s.w += v2.w;
      s.x += v3.x; s.y += v3.y; s.z += v3.z; s.w += v3.w;
    }
    for (; z < count; z += ZL) {
      const mnv_f4 v = *reinterpret_cast<const mnv_f4*>(part(z) + e);
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    if (ZL > 1) {
      __syncthreads();  // the previous pass has read its sums
      red[threadIdx.x] = s;
      __syncthreads();
      if (tz != 0) continue;
#pragma unroll
      for (int q = 1; q < ZL; ++q) {
        const mnv_f4 v = red[q * QL + tq];
        s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
      }
    }
    int m, n;
    mnv_partial_group_mn<T>(e / 4, m, n);
    m += m0;
    n += n0;
    if (m < prob.M) {
      if (n + 0 < prob.N) prob.c_store(m, n + 0, s.x);
      if (n + 1 < prob.N) prob.c_store(m, n + 1, s.y);
      if (n + 2 < prob.N) prob.c_store(m, n + 2, s.z);
      if (n + 3 < prob.N) prob.c_store(m, n + 3, s.w);
    }
  }
}

// Which tiles form the tail and into how many k ranges each is cut (z <= 1: none).  Only
// for launches of at least one large tile per CU (the device's count, mnv_cu_count) without k
// ranges of their own; taken when the uneven last tile per CU costs at least 3% (on 256 CUs:
// tiles / 256 = 2.64: 12%; 11.39: 5%; 3.96: 1%),
// with about three small workgroups per CU (two to four measured alike: conv2 data gradient
// 1.77 -> 1.74 / 1.71 / 1.70 ms, conv5 forward 0.71 -> 0.66 ms with any of them), at least
// eight slabs each, and only as far as the workspace holds the partial tiles.
struct MnvTailPlan {
  int begin, z;
};
static inline MnvTailPlan mnv_tail_plan(long long tiles, int slabs, size_t tile_floats,
                                        size_t ws_floats) {
  const int cus = mnv_cu_count();
  const MnvTailPlan none{(int)(tiles < 0x7fffffff ? tiles : 0x7fffffff), 1};
  if (tiles < cus || tiles > 0x3fffffff) return none;
  const int rem = (int)(tiles % cus);
  if (rem == 0) return none;
  const double per_cu = (double)tiles / cus, most = (double)((tiles + cus - 1) / cus);
  if ((most - per_cu) / most < 0.03) return none;
  int z = 3 * cus / rem;
  if (z > 16) z = 16;
  if (z > slabs / 8) z = slabs / 8;
  const size_t fit = ws_floats / ((size_t)rem * tile_floats);
  if ((size_t)z > fit) z = (int)fit;
  if (z < 2) return none;
  return MnvTailPlan{(int)(tiles - rem), z};
}

// Number of k ranges for `tiles` output tiles of `slabs` k-slabs each.  Workgroups are
// dealt evenly to the device's CUs, which hold four of them at a time, and the kernel ends when the
// fullest CU does: a split count that puts a few workgroups past a multiple of 1024 costs a
// whole extra round, so the estimate below (workgroups on the fullest CU x slabs each,
// corrected for the matrix pipe running below its rate with fewer than four workgroups in
// residence) is minimised rather than the count simply rounded up.
// `per_split` (optional) is what every additional k range costs for writing and re-reading
// its partial result, in the same unit (one slab of one workgroup); `cost_out` receives the
// estimate of the chosen count so that callers can compare tile shapes.
static inline int mnv_pick_splits(long long tiles, int slabs, int max_splits, double per_split = 0.0,
                                  double* cost_out = nullptr) {
  static const double rate[5] = {1.0, 0.45, 0.75, 0.92, 1.0};
  const int cus = mnv_cu_count();
  if (max_splits < 1) max_splits = 1;
  int best = 1;
  double best_cost = 0;
  for (int s = 1; s <= max_splits; ++s) {
    long long per_cu = (tiles * s + cus - 1) / cus;
    int len = (slabs + s - 1) / s;
    double cost = (double)per_cu * (len + 4) / rate[per_cu < 4 ? per_cu : 4] + (s > 1 ? per_split * s : 0.0);
    if (s == 1 || cost < best_cost * 0.98) {  // prefer fewer partial results on a near tie
      best = s;
      best_cost = cost;
    }
  }
  if (cost_out) *cost_out = best_cost;
  return best;
}

// Host-side launch of one tile configuration.  `splits` > 1 needs
// splits*M*N*sizeof(float) bytes at `workspace`.
// `tail_bytes`: bytes at `workspace` that a launch without k ranges may use for the partial
// tiles of its tail (0: never cut the tail).
template <class T, int G = 1, int PF = 1, class P>
static int mnv_gemm_launch(const P& prob, int splits, void* workspace, hipStream_t s,
                           size_t tail_bytes = 0) {
  const int tiles_m = (prob.M + T::BM - 1) / T::BM, tiles_n = (prob.N + T::BNU - 1) / T::BNU;
  const int total_slabs = prob.total_slabs;
  if (splits < 1) splits = 1;
  if (splits > total_slabs) splits = total_slabs > 0 ? total_slabs : 1;
  int per = (total_slabs + splits - 1) / splits;
  if (per < 1) per = 1;
  splits = total_slabs > 0 ? (total_slabs + per - 1) / per : 1;
  if ((long long)tiles_m * tiles_n > 0x7fffffffLL || splits > 65535) return MNV_ERR_INVALID;
  // The LDS limit of a kernel is an attribute per device; set once on each (idempotent: a
  // race only repeats the same call).
  static std::atomic<bool> attr_set[64];
  const size_t tile_bytes = G * T::lds_bytes(P::A_KFAST, P::B_KFAST);
  const size_t lds_limit = (G > 1 ? 160 : 64) * 1024;
  if (G > 1 && prob.extra_lds_bytes()) return MNV_ERR_INVALID;  // groups use every tile buffer
  if (tile_bytes + prob.extra_lds_bytes() > 48 * 1024) {
    int dev = 0;
    MNV_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64) return MNV_ERR_INVALID;
    if (!attr_set[dev].load(std::memory_order_acquire)) {
      MNV_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&mnv_gemm_kernel<T, P, G, false, PF>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_limit));
      attr_set[dev].store(true, std::memory_order_release);
    }
  }
  const size_t lds_bytes = tile_bytes + prob.extra_lds_bytes();
  if (lds_bytes > lds_limit) return MNV_ERR_INVALID;
  MnvTailPlan tail{tiles_m * tiles_n, 1};
  if (G == 1 && splits == 1 && T::MIN_WAVES == 4 && workspace && tail_bytes)
    tail = mnv_tail_plan((long long)tiles_m * tiles_n, total_slabs, (size_t)T::BM * T::BNU,
                         tail_bytes / sizeof(float));
  const int tail_tiles = tiles_m * tiles_n - tail.begin;
  hipLaunchKernelGGL((mnv_gemm_kernel<T, P, G, false, PF>),
                     dim3(tail.begin + tail_tiles * tail.z, 1, splits), dim3(T::NT * G), lds_bytes,
                     s, prob, tiles_m, tiles_n, per, reinterpret_cast<float*>(workspace),
                     tail.begin, tail.z);
  int rc = MNV_LAUNCH_STATUS();
  if (rc) return rc;
  if (tail.z > 1) {
    hipLaunchKernelGGL((mnv_gemm_tail_reduce_kernel<T, P>), dim3(T::BM * T::BNU / 1024, tail_tiles),
                       dim3(256), 0, s, prob, reinterpret_cast<const float*>(workspace), tiles_m,
                       tiles_n, tail.begin, tail.z);
    return MNV_LAUNCH_STATUS();
  }
  if (splits > 1) {
    // enough threads to cover the chip: one per element for a large output, up to 64 per
    // element (never more than half the ranges) for a small one
    const size_t mn = (size_t)prob.M * prob.N;
    const float* part = reinterpret_cast<const float*>(workspace);
    if (mn >= 65536 || splits < 8) rc = mnv_gemm_splitk_reduce_launch<P, 1>(prob, part, splits, s);
    else if (mn >= 16384 || splits < 32) rc = mnv_gemm_splitk_reduce_launch<P, 4>(prob, part, splits, s);
    else if (mn >= 4096 || splits < 128) rc = mnv_gemm_splitk_reduce_launch<P, 16>(prob, part, splits, s);
    else rc = mnv_gemm_splitk_reduce_launch<P, 64>(prob, part, splits, s);
  }
  return rc;
}

// Stream-k launch of one tile configuration (see mnv_gemm_kernel): as many workgroups as the
// current device holds at once, equal shares of the tiles x k-slabs, then the reduction.
// `*done` is false, and nothing was launched, when the plan does not apply: fewer than eight
// slabs per workgroup, more tiles than workgroups, or a workspace under
// mnv_gemm_streamk_bytes.  The plan depends on the extents, the device (its CU count and how
// many of the kernel's workgroups a CU holds) and nothing else.
template <class T>
static inline size_t mnv_gemm_streamk_bytes(long long tiles, int workgroups) {
  return (size_t)(workgroups + tiles) * T::BM * T::BNU * sizeof(float);
}

// `plan_workgroups` (optional): receives the number of workgroups of the plan, 0 when it
// does not apply, and nothing is launched.
template <class T, int PF = 1, class P>
static int mnv_gemm_streamk_launch(const P& prob, void* workspace, size_t ws_bytes, hipStream_t s,
                                   bool* done, int* plan_workgroups = nullptr) {
  *done = false;
  if (plan_workgroups) *plan_workgroups = 0;
  const int tiles_m = (prob.M + T::BM - 1) / T::BM, tiles_n = (prob.N + T::BNU - 1) / T::BNU;
  const long long tiles = (long long)tiles_m * tiles_n;
  const size_t lds_bytes = T::lds_bytes(P::A_KFAST, P::B_KFAST) + prob.extra_lds_bytes();
  if (!workspace || prob.total_slabs <= 0 || tiles > 0x7fffffffLL / prob.total_slabs ||
      lds_bytes > 64 * 1024)
    return MNV_OK;
  int dev = 0;
  MNV_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64) return MNV_ERR_INVALID;
  const void* fn = reinterpret_cast<const void*>(&mnv_gemm_kernel<T, P, 1, true, PF>);
  // (LDS bytes << 8 | workgroups per CU) of the last query on each device
  static std::atomic<unsigned long long> cached[64];
  static std::atomic<bool> attr_set[64];
  if (lds_bytes > 48 * 1024 && !attr_set[dev].load(std::memory_order_acquire)) {
    MNV_HIP_TRY(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024));
    attr_set[dev].store(true, std::memory_order_release);
  }
  unsigned long long c = cached[dev].load(std::memory_order_relaxed);
  if ((c >> 8) != lds_bytes || (c & 255) == 0) {
    int per_cu = 0;
    MNV_HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fn, T::NT, lds_bytes));
    if (per_cu < 1) return MNV_OK;
    if (per_cu > 255) per_cu = 255;
    c = ((unsigned long long)lds_bytes << 8) | (unsigned)per_cu;
    cached[dev].store(c, std::memory_order_relaxed);
  }
  const int workgroups = (int)(c & 255) * mnv_cu_count();
  if (tiles > workgroups || tiles * prob.total_slabs < 8LL * workgroups ||
      ws_bytes < mnv_gemm_streamk_bytes<T>(tiles, workgroups))
    return MNV_OK;
  // Aligned ranges per tile and the slabs of each (see mnv_gemm_kernel).  A range or a segment
  // costs about six slab times beside its slabs (first loads, the partial tile's store), and a
  // remaining workgroup works off tiles / left + 1 segments: the ranges are made that much
  // longer than an equal share, so that the remaining workgroups end with the others and not
  // after them.  When that leaves them nothing, they are not launched.
  const int aligned = (int)(workgroups / tiles);
  long long left = workgroups - tiles * aligned;
  int chunk = 0, rest = 0;
  if (left > 0) {
    chunk = (int)((tiles * (prob.total_slabs + 6LL) + workgroups - 1) / workgroups);
    rest = prob.total_slabs - aligned * chunk;
    if (rest <= 0) left = 0;
  }
  if (left == 0) {
    chunk = (prob.total_slabs + aligned - 1) / aligned;
    rest = 0;
  }
  const int launched = (int)(tiles * aligned + left);
  if (plan_workgroups) {
    *plan_workgroups = launched;
    *done = true;
    return MNV_OK;
  }
  hipLaunchKernelGGL((mnv_gemm_kernel<T, P, 1, true, PF>), dim3(launched), dim3(T::NT), lds_bytes, s,
                     prob, tiles_m, tiles_n, chunk, reinterpret_cast<float*>(workspace), aligned, 1);
  int rc = MNV_LAUNCH_STATUS();
  if (rc) return rc;
  // partial tiles per tile: the aligned ranges, and the remaining workgroups that met the tile
  const long long per_tile = aligned + (left ? left / tiles + 2 : 0);
  const float* part = reinterpret_cast<const float*>(workspace);
  const dim3 block(256);
  if (per_tile >= 64)
    hipLaunchKernelGGL((mnv_gemm_streamk_reduce_kernel<T, P, 16>),
                       dim3(T::BM * T::BNU / 64, (unsigned)tiles), block, 0, s, prob, part, tiles_m,
                       tiles_n, launched, aligned, rest);
  else if (per_tile >= 32)
    hipLaunchKernelGGL((mnv_gemm_streamk_reduce_kernel<T, P, 4>),
                       dim3(T::BM * T::BNU / 256, (unsigned)tiles), block, 0, s, prob, part, tiles_m,
                       tiles_n, launched, aligned, rest);
  else
    hipLaunchKernelGGL((mnv_gemm_streamk_reduce_kernel<T, P, 1>),
                       dim3(T::BM * T::BNU / 1024, (unsigned)tiles), block, 0, s, prob, part, tiles_m,
                       tiles_n, launched, aligned, rest);
  *done = true;
  return MNV_LAUNCH_STATUS();
}
#endif  // __HIPCC__
