// WTConv2d on the matrix cores of gfx950: plane-resident kernel for kernel sizes up to 5.
//
// Same layer maths as kernels2d.h (reference wtconv/wtconv2d.py:38-82), different arithmetic:
// every depthwise K x K convolution of the layer (base conv and the four sub-bands of every
// level) runs as v_mfma_f32_16x16x32_bf16 products.  A 4 x 4 block of outputs depends on an
// 8 x 8 patch of inputs (K <= 5), so for 16 blocks of one filter
//     D[16 outputs of a block][16 blocks] = Wt[16 outputs][64 patch elements] * Patch[64][16 blocks]
// is two MFMAs (patch rows 0-3 and 4-7).  Wt is the filter laid out as a Toeplitz matrix
// (39 % non-zero); the fold kernel writes it in the compact form the lanes pick their
// fragment from.  Lane (n = lane % 16, q = lane / 16) supplies row q (+4) of block n's patch
// -- 8 consecutive bf16 of an LDS row -- and receives outputs (row q, columns 0..3) of block n.
//
// Activations live in LDS as bf16 planes with a zero halo of 2.  bf16 tensors take one plane
// per buffer (NS = 1).  fp32 tensors are split into NS = 3 bf16 planes (v = h0 + h1 + h2
// exactly, 24 mantissa bits) and the folded weights likewise; the six products of total
// order <= 2 are accumulated in fp32, which leaves an error below that of an fp32 FMA chain.
// The Haar butterflies run unnormalised in fp32 (the factors 1/2 of analysis and synthesis
// are folded into the weights as 4^-level), coefficients are rounded (or split) to bf16 when
// they are written to LDS, accumulators, the partial reconstructions Z_l and the raw LL chain
// stay fp32.
#pragma once

#include "common.h"

namespace wt {

constexpr int kFragEntries = 21;     // 5 kernel rows x 4 column shifts, then one all-zero entry
constexpr int kMfmaBlock = 256;
constexpr int kDivShift = 20;        // magic reciprocals: exact for dividends < 4096, divisors <= 256

struct MPlan {
  int B, C, H, W, L;
  int pb, upc, nunits;               // planes (one channel, consecutive batch items) per unit; units per channel; total
  int bq, br;                        // B = upc * bq + br: the first br units of a channel take bq + 1 batch items, the rest bq
  int nfilt;                         // 1 + 4 L
  int h[kMaxLevels + 1], w[kMaxLevels + 1];        // extent of level l (0 = pixels)
  int nbr[kMaxLevels + 1], nbc[kMaxLevels + 1];    // 4x4 blocks per plane: rows, columns
  int bpp[kMaxLevels + 1], nblk[kMaxLevels + 1];   // blocks per plane, per unit
  unsigned mg_bpp0, mg_nbc0;                                 // reciprocals of bpp[0], nbc[0]
  unsigned mg_hw[kMaxLevels + 1], mg_w[kMaxLevels + 1];      // reciprocals of h*w, w
  // MFMA tiles: 16 blocks = TR block-rows x TC block-columns, TC = 2^tcs >= nbc; the block-rows of
  // the stacked planes of a unit are numbered R = p * nbr + bi
  int tcs[kMaxLevels + 1], nrow[kMaxLevels + 1], ntile[kMaxLevels + 1];
  int rtoff[kMaxLevels + 1];         // byte offset of the block-row table of level l
  int pitch[kMaxLevels + 1];         // LDS row pitch of a level-l plane in bf16 elements (multiple of 4)
  int prows[kMaxLevels + 1];         // LDS rows from one stacked plane to the next: 4 nbr + 2
  int aoff[kMaxLevels + 1];          // byte offset of (slot 0, row -2, column -2) of sub-band 0, split 0
  int asub[kMaxLevels + 1];          // bytes from one plane stack to the next (sub-bands, then splits)
  int zoff[kMaxLevels + 2], zpitch[kMaxLevels + 2], zpl[kMaxLevels + 2];   // fp32 Z_l, l = 1..L
  int lloff[kMaxLevels + 1], llpl[kMaxLevels + 1];                         // fp32 raw LL of level l, 2 <= l < L
  int toff;                          // byte offset of the fragment table of the current channel ...
  int tfirst;                        // ... which starts at this filter (the filters before it live in registers)
  int lds_bytes;
};

// ------------------------------------------------------------------------------ planning
// Reciprocal for fast_div(): exact for every dividend in [0, maxv], or the shape is refused.
constexpr bool make_magic(int d, int maxv, unsigned* magic) {
  if (d < 1 || maxv >= 4096) return false;
  const unsigned m = ((1u << kDivShift) + d - 1) / d;
  if (m >= (1u << 24)) return false;
  for (int v = 0; v <= maxv; ++v)
    if (static_cast<int>((static_cast<unsigned long long>(v) * m) >> kDivShift) != v / d) return false;
  *magic = m;
  return true;
}

// Everything of a plan that depends on the plane shape, the levels, the split count and the
// planes per unit only (not on batch or channels); false if the kernel cannot index the shape.
// constexpr: the kernels of the common shapes take it as a compile-time constant.
constexpr bool make_mplan_geometry(int H, int W, int L, int NS, int pb, MPlan* out) {
  auto cdiv = [](int a, int b) { return (a + b - 1) / b; };
  auto rup = [](int v, int m) { return (v + m - 1) / m * m; };
  MPlan pl = {};
  pl.H = H; pl.W = W; pl.L = L;
  pl.pb = pb;
  pl.nfilt = 1 + 4 * L;
  pl.h[0] = H; pl.w[0] = W;
  for (int l = 1; l <= L; ++l) { pl.h[l] = (pl.h[l - 1] + 1) / 2; pl.w[l] = (pl.w[l - 1] + 1) / 2; }
  int off = 0;
  pl.toff = off;
  pl.tfirst = NS == 1 ? 5 : 0;       // one split plane: base conv and level 1 stay in registers
  off += NS * (pl.nfilt - pl.tfirst) * kFragEntries * 16;
  for (int l = 0; l <= L; ++l) {
    pl.nbr[l] = cdiv(pl.h[l], 4);
    pl.nbc[l] = cdiv(pl.w[l], 4);
    pl.bpp[l] = pl.nbr[l] * pl.nbc[l];
    pl.nblk[l] = pb * pl.bpp[l];
    pl.pitch[l] = 4 * pl.nbc[l] + 4;
    pl.prows[l] = 4 * pl.nbr[l] + 2;
    if (l == 0) {
      if (!make_magic(pl.bpp[0], pl.nblk[0] + kMfmaBlock * 4, &pl.mg_bpp0)) return false;
      if (!make_magic(pl.nbc[0], pl.bpp[0], &pl.mg_nbc0)) return false;
    }
    pl.tcs[l] = 0;
    while ((1 << pl.tcs[l]) < pl.nbc[l]) ++pl.tcs[l];
    if (pl.tcs[l] > 4) return false;                 // planes wider than 64 are not tiled
    pl.nrow[l] = pb * pl.nbr[l];
    pl.ntile[l] = cdiv(pl.nrow[l], 16 >> pl.tcs[l]);
    if (pb * pl.prows[l] + 8 >= 4096 || pb > 255 || pl.nbr[l] >= 4096) return false;   // block-row table fields
    if (l >= 3) {
      if (!make_magic(pl.h[l] * pl.w[l], pb * pl.h[l] * pl.w[l] + kMfmaBlock, &pl.mg_hw[l])) return false;
      if (!make_magic(pl.w[l], pl.h[l] * pl.w[l], &pl.mg_w[l])) return false;
    }
    pl.aoff[l] = off;
    pl.asub[l] = rup((pb * pl.prows[l] + 2) * pl.pitch[l] * 2, 16);
    off += pl.asub[l] * NS * (l == 0 ? 1 : 4);
    if (off > (1 << 20)) return false;
  }
  for (int l = 1; l <= L; ++l) {
    pl.zpitch[l] = 4 * pl.nbc[l - 1];
    pl.zpl[l] = 4 * pl.nbr[l - 1] * pl.zpitch[l];
    pl.zoff[l] = off;
    int zbytes = pb * pl.zpl[l] * 4;
    const int staging = NS * pl.tfirst * kFragEntries * 16;      // Z_1 doubles as staging area when a channel's parameters are folded
    if (l == 1 && zbytes < staging) zbytes = staging;
    off += zbytes;
    if (off > (1 << 20)) return false;
  }
  for (int l = 2; l < L; ++l) {
    pl.llpl[l] = pl.h[l] * pl.w[l];
    pl.lloff[l] = off;
    off += rup(pb * pl.llpl[l] * 4, 16);
  }
  for (int l = 0; l <= L; ++l) {
    pl.rtoff[l] = off;
    off += rup(pl.nrow[l] * 4, 16);
  }
  off += 256;      // lanes beyond a plane's last block column read a few elements past its rows
  pl.lds_bytes = rup(off, 16);
  *out = pl;
  return true;
}

// Where a kernel takes the shape-dependent part of its plan from: the kernel argument, or a
// compile-time constant (every LDS offset then folds into the instructions).
struct GeoRuntime {
  static constexpr bool kStatic = false;
  static constexpr int kL = 0;
};
template <int H, int W, int L, int PB>
struct GeoStatic {
  static constexpr bool kStatic = true;
  static constexpr int kL = L;
  template <int NS> static constexpr MPlan plan() {
    MPlan p = {};
    make_mplan_geometry(H, W, L, NS, PB, &p);
    return p;
  }
};

// f(l) for l = LO..L (upwards) / L..LO (downwards).  With a static geometry the calls are
// separate instantiations with a constant level, so that every per-level plan field folds; a
// level that is only known at run time would force the constant plan into scratch memory.
template <typename Geo, int LO, typename F>
__device__ __forceinline__ void levels_up(int L, F&& f) {
  if constexpr (Geo::kStatic) {
    using std::integral_constant;
    if constexpr (LO <= 0) f(integral_constant<int, 0>{});
    if constexpr (LO <= 1 && Geo::kL >= 1) f(integral_constant<int, 1>{});
    if constexpr (LO <= 2 && Geo::kL >= 2) f(integral_constant<int, 2>{});
    if constexpr (LO <= 3 && Geo::kL >= 3) f(integral_constant<int, 3>{});
    if constexpr (LO <= 4 && Geo::kL >= 4) f(integral_constant<int, 4>{});
    if constexpr (LO <= 5 && Geo::kL >= 5) f(integral_constant<int, 5>{});
  } else {
#pragma unroll 1
    for (int l = LO; l <= L; ++l) f(l);
  }
}
template <typename Geo, int LO, typename F>
__device__ __forceinline__ void levels_down(int L, F&& f) {
  if constexpr (Geo::kStatic) {
    using std::integral_constant;
    if constexpr (LO <= 5 && Geo::kL >= 5) f(integral_constant<int, 5>{});
    if constexpr (LO <= 4 && Geo::kL >= 4) f(integral_constant<int, 4>{});
    if constexpr (LO <= 3 && Geo::kL >= 3) f(integral_constant<int, 3>{});
    if constexpr (LO <= 2 && Geo::kL >= 2) f(integral_constant<int, 2>{});
    if constexpr (LO <= 1 && Geo::kL >= 1) f(integral_constant<int, 1>{});
  } else {
#pragma unroll 1
    for (int l = L; l >= LO; --l) f(l);
  }
}

// -------------------------------------------------------------------------------- helpers
struct Frag { uint32_t d[4]; };      // 8 bf16
struct Acc { float v[4]; };

__device__ __forceinline__ void mfma_bf16(const Frag& a, const Frag& b, Acc& c) {
#ifdef WT_EMULATE
  uint16_t ua[8], ub[8];
  for (int i = 0; i < 4; ++i) {
    ua[2 * i] = static_cast<uint16_t>(a.d[i]); ua[2 * i + 1] = static_cast<uint16_t>(a.d[i] >> 16);
    ub[2 * i] = static_cast<uint16_t>(b.d[i]); ub[2 * i + 1] = static_cast<uint16_t>(b.d[i] >> 16);
  }
  ::emu::mfma_16x16x32_bf16(ua, ub, c.v);
#else
  typedef __bf16 wt_bf16x8 __attribute__((ext_vector_type(8)));
  typedef float wt_f32x4 __attribute__((ext_vector_type(4)));
  typedef uint32_t wt_u32x4 __attribute__((ext_vector_type(4)));
  const wt_u32x4 au = {a.d[0], a.d[1], a.d[2], a.d[3]}, bu = {b.d[0], b.d[1], b.d[2], b.d[3]};
  wt_f32x4 cv = {c.v[0], c.v[1], c.v[2], c.v[3]};
  cv = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(wt_bf16x8, au), __builtin_bit_cast(wt_bf16x8, bu),
                                               cv, 0, 0, 0);
  c.v[0] = cv[0]; c.v[1] = cv[1]; c.v[2] = cv[2]; c.v[3] = cv[3];
#endif
}

// Orders the LDS traffic of one wave inside code that only some waves of the workgroup run.
#ifdef WT_EMULATE
#define WT_WAVE_SYNC_DIVERGENT() ::emu::wave_barrier()
#else
#define WT_WAVE_SYNC_DIVERGENT() WT_WAVE_LDS_SYNC()
#endif

template <typename V> __device__ __forceinline__ V lds_ld(const char* lds, int off) {
  return *reinterpret_cast<const V*>(lds + off);
}
template <typename V> __device__ __forceinline__ void lds_st(char* lds, int off, V v) {
  *reinterpret_cast<V*>(lds + off) = v;
}

// 8 consecutive bf16 at an 8-byte aligned LDS offset
__device__ __forceinline__ Frag lds_frag8(const char* lds, int off) {
  const uint2 lo = lds_ld<uint2>(lds, off), hi = lds_ld<uint2>(lds, off + 8);
  Frag f; f.d[0] = lo.x; f.d[1] = lo.y; f.d[2] = hi.x; f.d[3] = hi.y;
  return f;
}
// ... at a 16-byte aligned offset (fragment table)
__device__ __forceinline__ Frag lds_frag16(const char* lds, int off) {
  const uint4 v = lds_ld<uint4>(lds, off);
  Frag f; f.d[0] = v.x; f.d[1] = v.y; f.d[2] = v.z; f.d[3] = v.w;
  return f;
}

__device__ __forceinline__ int fast_div(int v, unsigned magic) {
#ifdef WT_EMULATE
  return static_cast<int>((static_cast<uint64_t>(static_cast<unsigned>(v)) * magic) >> kDivShift);
#else
  return static_cast<int>(__umul24(static_cast<unsigned>(v), magic) >> kDivShift);
#endif
}

// Two floats -> NS words of two bf16 each whose sum is the pair (exactly, for NS = 3).
template <int NS>
__device__ __forceinline__ void split_pair(float lo, float hi, uint32_t (&w)[NS]) {
#pragma unroll
  for (int j = 0; j < NS; ++j) {
    w[j] = pack_bf16x2(lo, hi);
    if (j + 1 < NS) {
      lo -= __uint_as_float(w[j] << 16);
      hi -= __uint_as_float(w[j] & 0xffff0000u);
    }
  }
}

// ------------------------------------------------------------------ fragment table (fold)
// Entry e = 4 kh + cs of filter f of channel c: kernel row kh of the filter (embedded in 5 x 5,
// scaled by gamma and 4^-level, rotated by 180 degrees when flip != 0) shifted right by cs in a
// window of 8 -- the 8 bf16 a lane feeds the MFMA with -- as NS split words; entry 20 is zero.
// Filter 0 is the base conv, filter 1 + 4 (l - 1) + s sub-band s of level l.
template <int NS>
__device__ __forceinline__ void fold_entry(const ParamTable& p, int pdtype, int K, int flip, int c, int f, int e,
                                           uint4 (&out)[NS]) {
  const int KK = K * K, o = 2 - K / 2;
  float v[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = 0.f;
  if (e < 20) {
    const int kh = e >> 2, cs = e & 3;
    const int ih = kh - o;
    float scale;
    const void* wp;
    int ch;
    if (f == 0) {
      wp = p.base_weight; ch = c;
      scale = load_param(p.base_scale, pdtype, c);
    } else {
      const int l = (f - 1) >> 2, s = (f - 1) & 3;
      wp = p.wt_weight[l]; ch = c * 4 + s;
      scale = load_param(p.wt_scale[l], pdtype, ch);
#pragma unroll 1
      for (int i = 0; i <= l; ++i) scale *= 0.25f;
    }
    // the (up to five) taps of the entry's kernel row, fetched together whether or not the entry uses them: loads
    // behind per-tap conditions would complete one after the other, and a channel switch waits for this fold
    const bool row_ok = ih >= 0 && ih < K;
    const int frow = row_ok ? (flip ? K - 1 - ih : ih) : 0;
    const int rowi = ch * KK + frow * K;
    float wr[5];
    if (pdtype == WTCONV_F32) {
      const float* w = static_cast<const float*>(wp) + rowi;
#pragma unroll
      for (int i = 0; i < 5; ++i) wr[i] = w[i < K ? i : K - 1];
    } else {
      const uint16_t* w = static_cast<const uint16_t*>(wp) + rowi;
      uint16_t h[5];
#pragma unroll
      for (int i = 0; i < 5; ++i) h[i] = w[i < K ? i : K - 1];
#pragma unroll
      for (int i = 0; i < 5; ++i) wr[i] = pdtype == WTCONV_F16 ? f16_bits_to_f32(h[i]) : bf16_to_f32(h[i]);
    }
    if (row_ok) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int iw = j - cs - o;
        if (iw >= 0 && iw < K && j - cs < 5 && j - cs >= 0) {
          const int fi = flip ? K - 1 - iw : iw;
          float t = wr[0];
#pragma unroll
          for (int i = 1; i < 5; ++i) t = fi == i ? wr[i] : t;
          v[j] = t * scale;
        }
      }
    }
  }
#pragma unroll
  for (int js = 0; js < NS; ++js) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      w[i] = pack_bf16x2(v[2 * i], v[2 * i + 1]);
      v[2 * i] -= __uint_as_float(w[i] << 16);
      v[2 * i + 1] -= __uint_as_float(w[i] & 0xffff0000u);
    }
    out[js].x = w[0]; out[js].y = w[1]; out[js].z = w[2]; out[js].w = w[3];
  }
}

// ------------------------------------------------------------------ pixel blocks in registers
template <typename T> struct PixRow;
template <> struct PixRow<float> { float4 v; };
template <> struct PixRow<bf16_t> { uint2 v; };
// Rows of bf16 planes that are not whole aligned vectors still move as one 8-byte access per row of a block: global
// memory takes unaligned accesses (the compiler itself emits one dwordx2 for an 8-byte copy from a 2-byte aligned
// address).  Columns past the row end come along and are cleared before use; nothing is computed on the loaded
// words before the commit, so all the loads of a block stay in flight.
__device__ __forceinline__ void pix_load4u(uint2& v, const bf16_t* p) { __builtin_memcpy(&v, p, 8); }
__device__ __forceinline__ void pix_store4u(bf16_t* p, const uint2& v) { __builtin_memcpy(p, &v, 8); }
// words that keep the valid columns of a block row: bits 4..7 of `cmask` say which of its four columns exist
__device__ __forceinline__ uint2 pix_col_mask(unsigned cmask) {
  uint2 m;
  m.x = ((cmask & 16u) ? 0x0000ffffu : 0u) | ((cmask & 32u) ? 0xffff0000u : 0u);
  m.y = ((cmask & 64u) ? 0x0000ffffu : 0u) | ((cmask & 128u) ? 0xffff0000u : 0u);
  return m;
}

__device__ __forceinline__ void pix_zero(PixRow<float>& r) { r.v.x = r.v.y = r.v.z = r.v.w = 0.f; }
__device__ __forceinline__ void pix_zero(PixRow<bf16_t>& r) { r.v.x = r.v.y = 0u; }
__device__ __forceinline__ void pix_load4(PixRow<float>& r, const float* p) { r.v = *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ void pix_load4(PixRow<bf16_t>& r, const bf16_t* p) { r.v = *reinterpret_cast<const uint2*>(p); }
__device__ __forceinline__ void pix_set(PixRow<float>& r, int i, float v) {
  if (i == 0) r.v.x = v; else if (i == 1) r.v.y = v; else if (i == 2) r.v.z = v; else r.v.w = v;
}
__device__ __forceinline__ void pix_set(PixRow<bf16_t>& r, int i, bf16_t v) {
  const uint32_t u = static_cast<uint32_t>(v) << ((i & 1) * 16);
  if (i < 2) r.v.x |= u; else r.v.y |= u;
}
// the four bf16 of a row as two packed words
__device__ __forceinline__ uint2 pix_words(const PixRow<bf16_t>& r) { return r.v; }
__device__ __forceinline__ uint2 pix_words(const PixRow<float>&) { uint2 w; w.x = w.y = 0u; return w; }   // (never taken)
__device__ __forceinline__ void pix_get(const PixRow<float>& r, float (&f)[4]) {
  f[0] = r.v.x; f[1] = r.v.y; f[2] = r.v.z; f[3] = r.v.w;
}
__device__ __forceinline__ void pix_get(const PixRow<bf16_t>& r, float (&f)[4]) {
  f[0] = __uint_as_float(r.v.x << 16); f[1] = __uint_as_float(r.v.x & 0xffff0000u);
  f[2] = __uint_as_float(r.v.y << 16); f[3] = __uint_as_float(r.v.y & 0xffff0000u);
}

// Block-row table entry: LDS row of the block-row's first patch row | plane slot << 12 | block-row in the plane << 20.
__device__ __forceinline__ unsigned rowtab_entry(int rowidx, int p, int bi) {
  return static_cast<unsigned>(rowidx) | (static_cast<unsigned>(p) << 12) | (static_cast<unsigned>(bi) << 20);
}

template <int NS>
__device__ __forceinline__ void load_b(const char* lds, int boff, int bsplit, int row4, Frag (&bt)[NS], Frag (&bb)[NS]) {
#pragma unroll
  for (int j = 0; j < NS; ++j) {
    bt[j] = lds_frag8(lds, boff + j * bsplit);
    bb[j] = lds_frag8(lds, boff + j * bsplit + row4);
  }
}

// Toeplitz fragments of one filter: `tab` = byte offset of the filter's table in split 0.
template <int NS>
__device__ __forceinline__ void load_a(const char* lds, int tab, int tsplit, int ent_top, int ent_bot,
                                       Frag (&at)[NS], Frag (&ab)[NS]) {
#pragma unroll
  for (int j = 0; j < NS; ++j) {
    at[j] = lds_frag16(lds, tab + j * tsplit + ent_top * 16);
    ab[j] = lds_frag16(lds, tab + j * tsplit + ent_bot * 16);
  }
}

// acc += Wt * Patch over both patch halves: all split products of total order < NS, smallest terms first.
template <int NS>
__device__ __forceinline__ void mma_tile(const Frag (&at)[NS], const Frag (&ab)[NS], const Frag (&bt)[NS],
                                         const Frag (&bb)[NS], Acc& acc) {
#pragma unroll
  for (int order = NS - 1; order >= 0; --order)
#pragma unroll
    for (int js = 0; js <= order; ++js) {
      const int jw = order - js;
      mfma_bf16(at[jw], bt[js], acc);
      mfma_bf16(ab[jw], bb[js], acc);
    }
}

// Inverse Haar butterfly (unnormalised) of four coefficients per sub-band: two rows of 8.
__device__ __forceinline__ void synth_rows(const Acc (&a)[4], float (&top)[8], float (&bot)[8]) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float s1 = a[0].v[j] + a[1].v[j], d1 = a[0].v[j] - a[1].v[j];
    const float s2 = a[2].v[j] + a[3].v[j], d2 = a[2].v[j] - a[3].v[j];
    top[2 * j] = s1 + s2; top[2 * j + 1] = s1 - s2;
    bot[2 * j] = d1 + d2; bot[2 * j + 1] = d1 - d2;
  }
}

// Lane's share of tile T at one level: which block (plane slot p, block-row bi, block-column tc)
// and where its patch row q starts.
struct TileLane {
  int boff, p, bi, tc;
  bool valid;
};
__device__ __forceinline__ TileLane tile_lane(const char* lds, int T, int n, int q, int tcs, int nrow, int nbc,
                                              int rtoff, int aoff, int pitch_bytes) {
  TileLane t;
  t.tc = n & ((1 << tcs) - 1);
  const int R = (T << (4 - tcs)) + (n >> tcs);
  t.valid = R < nrow && t.tc < nbc;
  const unsigned e = lds_ld<uint32_t>(lds, rtoff + 4 * (R < nrow ? R : nrow - 1));
  t.p = static_cast<int>((e >> 12) & 0xffu);
  t.bi = static_cast<int>(e >> 20);
  t.boff = aoff + imul(static_cast<int>(e & 0xfffu) + q, pitch_bytes) + 8 * t.tc;
  return t;
}

// ------------------------------------------------------------------------------ the kernel
// Grid: persistent workgroups, each takes a contiguous range of units (pb planes of one
// channel).  NBL: 4x4 pixel blocks a thread loads per unit.  VEC: plane rows are whole,
// aligned 4-element vectors.  RES: the Toeplitz fragments of the base conv and of level 1 stay
// in registers while the channel does not change.
template <typename T, int NS, int NBL, bool VEC, bool RES, typename Geo>
__global__ void __launch_bounds__(kMfmaBlock, NS == 1 ? 4 : 2)      // waves per SIMD the register budget must allow
wt2d_mfma_kernel(const T* __restrict__ x, T* __restrict__ out, const ParamTable prm, int pdtype, int K, int flip,
                 int use_bias, const MPlan plarg, unsigned* __restrict__ zero_words, int nzero) {
  // the plan: shape-dependent fields from the compile-time constant where there is one
  const MPlan pl = [&]() {
    if constexpr (Geo::kStatic) {
      constexpr MPlan g = Geo::template plan<NS>();
      MPlan p = g;
      p.B = plarg.B; p.C = plarg.C; p.upc = plarg.upc; p.nunits = plarg.nunits; p.bq = plarg.bq; p.br = plarg.br;
      return p;
    } else {
      return plarg;
    }
  }();
  WT_SHARED_FLOATS(ldsf);
  char* lds = reinterpret_cast<char*>(ldsf);
  const int tid = threadIdx.x, lane = tid & 63, wave = WT_UNIFORM(tid >> 6);
  const int n = lane & 15, q = lane >> 4;
  const int L = pl.L, H = pl.H, W = pl.W;
  const int HW = H * W;
  // the channel tickets of a parameter-gradient pass that follows on the stream
  if (blockIdx.x == 0)
    for (int i = tid; i < nzero; i += kMfmaBlock) zero_words[i] = 0u;

  // Toeplitz fragment entries of this lane: output (row ar, column ac) of a block, patch row q (+4)
  const int ar = n >> 2, ac = n & 3;
  const int ent_top = (q - ar >= 0) ? (q - ar) * 4 + ac : 20;
  const int ent_bot = (q - ar <= 0) ? (4 + q - ar) * 4 + ac : 20;
  const int tsplit = (pl.nfilt - pl.tfirst) * kFragEntries * 16;      // bytes between the split tables in LDS

  for (int o = tid * 16; o < pl.lds_bytes; o += kMfmaBlock * 16) {
    uint4 z; z.x = z.y = z.z = z.w = 0u;
    lds_st<uint4>(lds, o, z);
  }
  WT_LDS_BARRIER();
  levels_up<Geo, 0>(L, [&](auto lc) {
    const int l = lc;
    for (int R = tid; R < pl.nrow[l]; R += kMfmaBlock) {
      const int p = R / pl.nbr[l], bi = R - p * pl.nbr[l];
      lds_st<uint32_t>(lds, pl.rtoff[l] + 4 * R, rowtab_entry(p * pl.prows[l] + 4 * bi, p, bi));
    }
  });

  // ---- per-thread constants of the commit role: which 4x4 pixel blocks this thread owns
  int c_goff[NBL], c_x0[NBL], c_a1[NBL], c_a2[NBL], c_ll[NBL], c_p[NBL];
  unsigned c_mask[NBL];      // bits 0-3: rows inside the plane; bits 4-7: columns inside; bit 8: block exists
#pragma unroll
  for (int i = 0; i < NBL; ++i) {
    const int g = tid + kMfmaBlock * i;
    const bool act = g < pl.nblk[0];
    const int gg = act ? g : 0;
    const int p = fast_div(gg, pl.mg_bpp0);
    const int rem = gg - imul(p, pl.bpp[0]);
    const int bi = fast_div(rem, pl.mg_nbc0);
    const int bj = rem - imul(bi, pl.nbc[0]);
    unsigned m = act ? 0x100u : 0u;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      if (4 * bi + r < H) m |= 1u << r;
      if (4 * bj + r < W) m |= 16u << r;
    }
    c_mask[i] = m;
    c_p[i] = p;
    c_goff[i] = p * pl.C * HW + 4 * bi * W + 4 * bj;
    c_x0[i] = pl.aoff[0] + ((p * pl.prows[0] + 4 * bi + 2) * pl.pitch[0] + 4 * bj + 2) * 2;
    c_a1[i] = pl.aoff[1] + ((p * pl.prows[1] + 2 * bi + 2) * pl.pitch[1] + 2 * bj + 2) * 2;
    c_a2[i] = L >= 2 ? pl.aoff[2] + ((p * pl.prows[2] + bi + 2) * pl.pitch[2] + bj + 2) * 2 : 0;
    c_ll[i] = L >= 3 ? pl.lloff[2] + (p * pl.llpl[2] + bi * pl.w[2] + bj) * 4 : 0;
  }
  // plan fields of the two finest levels, used in every unit
  const int asub0 = pl.asub[0], asub1 = pl.asub[1], asub2 = pl.asub[2];
  const int pitchB0 = pl.pitch[0] * 2, pitchB1 = pl.pitch[1] * 2;
  const int aoff0 = pl.aoff[0], aoff1 = pl.aoff[1];
  const int tcs0 = pl.tcs[0], tcs1 = pl.tcs[1], nrow0 = pl.nrow[0], nrow1 = pl.nrow[1];
  const int nbc0 = pl.nbc[0], nbc1 = pl.nbc[1], ntile0 = pl.ntile[0], ntile1 = pl.ntile[1];
  const int rtoff0 = pl.rtoff[0], rtoff1 = pl.rtoff[1];
  const int zoff1 = pl.zoff[1], zpitch1 = pl.zpitch[1], zpl1 = pl.zpl[1];
  const int zoff2 = pl.zoff[2], zpitch2 = pl.zpitch[2], zpl2 = pl.zpl[2];
  const int toff = pl.toff, upc = pl.upc, pb = pl.pb, C = pl.C, B = pl.B;

  const int G = gridDim.x;
  const int wg = xcd_contiguous(blockIdx.x, G);
  const int u_begin = static_cast<int>(static_cast<long long>(wg) * pl.nunits / G);
  const int u_end = static_cast<int>(static_cast<long long>(wg + 1) * pl.nunits / G);

  PixRow<T> pf[NBL][4];
  const size_t total_elems = static_cast<size_t>(B) * C * HW;
  auto fetch = [&](int u) {
    const int c = u / upc;
    const int ubf = u - c * upc;
    const int b0 = ubf * pl.bq + (ubf < pl.br ? ubf : pl.br);      // the batch is spread evenly over the channel's units (see below)
    const size_t base_off = (static_cast<size_t>(b0) * C + c) * HW;
    const T* base = x + base_off;
#pragma unroll
    for (int i = 0; i < NBL; ++i) {
      const bool plane_ok = (c_mask[i] & 0x100u) && c_p[i] < pl.bq + (ubf < pl.br ? 1 : 0);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        pix_zero(pf[i][r]);
        if (plane_ok && (c_mask[i] >> r & 1u)) {
          const T* src = base + c_goff[i] + r * W;
          if constexpr (VEC) {
            if (c_mask[i] & 16u) pix_load4(pf[i][r], src);
          } else if constexpr (sizeof(T) == 2) {
            // one unaligned 8-byte load per row (columns past the row end are cleared at the commit); only a row
            // whose four elements would reach past the end of the tensor goes element by element
            if (base_off + c_goff[i] + r * W + 4 <= total_elems) {
              pix_load4u(pf[i][r].v, src);
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (c_mask[i] >> (4 + e) & 1u) pix_set(pf[i][r], e, src[e]);
            }
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (c_mask[i] >> (4 + e) & 1u) pix_set(pf[i][r], e, src[e]);
          }
        }
      }
    }
  };
  if (u_begin < u_end) fetch(u_begin);

  constexpr int NR = RES ? NS : 1;
  Frag ra0t[NR], ra0b[NR], ra1t[4][NR], ra1b[4][NR];     // resident fragments (RES only)
  int cur_c = -1;
  float bias = 0.f;
#pragma unroll 1
  for (int u = u_begin; u < u_end; ++u) {
    const int c = u / upc;
    // The batch is spread evenly over the units of a channel: at most pb items each, all units within one plane of
    // each other (a short last unit would leave the workgroups that get it with less work than the rest).
    const int ub = u - c * upc;
    const int b0 = ub * pl.bq + (ub < pl.br ? ub : pl.br);
    const int np = pl.bq + (ub < pl.br ? 1 : 0);   // planes of this unit that exist
    if (c != cur_c) {     // (the previous unit ended with a barrier: nobody still reads the old table)
      // fold this channel's parameters into the fragment table: filters from `tfirst` on into their
      // LDS table, the ones before it (held in registers) through the idle Z_1 buffer
      const int nent = pl.nfilt * kFragEntries;
      const int nf_lds = (pl.nfilt - pl.tfirst) * kFragEntries;
      for (int i = tid; i < nent; i += kMfmaBlock) {
        const int f = i / kFragEntries, e = i - f * kFragEntries;
        uint4 w[NS];
        fold_entry<NS>(prm, pdtype, K, flip, c, f, e, w);
#pragma unroll
        for (int j = 0; j < NS; ++j) {
          const int o = f >= pl.tfirst ? toff + (j * nf_lds + i - pl.tfirst * kFragEntries) * 16 : zoff1 + (j * pl.tfirst * kFragEntries + i) * 16;
          lds_st<uint4>(lds, o, w[j]);
        }
      }
      bias = (use_bias && prm.base_bias != nullptr)
                 ? load_param(prm.base_bias, pdtype, c) * load_param(prm.base_scale, pdtype, c) : 0.f;
      cur_c = c;
      if constexpr (RES) {
        WT_LDS_BARRIER();
        ra0t[0] = lds_frag16(lds, zoff1 + ent_top * 16);
        ra0b[0] = lds_frag16(lds, zoff1 + ent_bot * 16);
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          ra1t[s][0] = lds_frag16(lds, zoff1 + ((1 + s) * kFragEntries + ent_top) * 16);
          ra1b[s][0] = lds_frag16(lds, zoff1 + ((1 + s) * kFragEntries + ent_bot) * 16);
        }
      }
    }

    // ---- commit: pixels -> level-0 planes; analysis levels 1 and 2 from registers
#pragma unroll
    for (int i = 0; i < NBL; ++i) {
      if (!(c_mask[i] & 0x100u)) continue;
      float v[4][4];
      if constexpr (!VEC && sizeof(T) == 2) {      // clear the columns that came along from past the row end
        const uint2 m = pix_col_mask(c_mask[i]);
#pragma unroll
        for (int r = 0; r < 4; ++r) { pf[i][r].v.x &= m.x; pf[i][r].v.y &= m.y; }
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) pix_get(pf[i][r], v[r]);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        uint32_t w0[NS], w1[NS];
        if constexpr (NS == 1 && sizeof(T) == 2) {
          const uint2 w = pix_words(pf[i][r]);      // the values are bf16 already
          w0[0] = w.x;
          w1[0] = w.y;
        } else {
          split_pair<NS>(v[r][0], v[r][1], w0);
          split_pair<NS>(v[r][2], v[r][3], w1);
        }
#pragma unroll
        for (int j = 0; j < NS; ++j) {
          const int o = c_x0[i] + j * asub0 + r * pitchB0;
          lds_st<uint32_t>(lds, o, w0[j]);
          lds_st<uint32_t>(lds, o + 4, w1[j]);
        }
      }
      float ll1[2][2];
#pragma unroll
      for (int i2 = 0; i2 < 2; ++i2) {
        float cf[4][2];
#pragma unroll
        for (int j2 = 0; j2 < 2; ++j2) {
          const float a = v[2 * i2][2 * j2], b = v[2 * i2][2 * j2 + 1];
          const float cc = v[2 * i2 + 1][2 * j2], d = v[2 * i2 + 1][2 * j2 + 1];
          const float s1 = a + b, d1 = a - b, s2 = cc + d, d2 = cc - d;
          cf[0][j2] = s1 + s2; cf[1][j2] = s1 - s2; cf[2][j2] = d1 + d2; cf[3][j2] = d1 - d2;
        }
        ll1[i2][0] = cf[0][0]; ll1[i2][1] = cf[0][1];
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          uint32_t w[NS];
          split_pair<NS>(cf[s][0], cf[s][1], w);
#pragma unroll
          for (int j = 0; j < NS; ++j)
            lds_st<uint32_t>(lds, c_a1[i] + (j * 4 + s) * asub1 + i2 * pitchB1, w[j]);
        }
      }
      if (L >= 2) {
        const float a = ll1[0][0], b = ll1[0][1], cc = ll1[1][0], d = ll1[1][1];
        const float s1 = a + b, d1 = a - b, s2 = cc + d, d2 = cc - d;
        const float cf[4] = {s1 + s2, s1 - s2, d1 + d2, d1 - d2};
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          uint32_t w[NS];
          split_pair<NS>(cf[s], 0.f, w);
#pragma unroll
          for (int j = 0; j < NS; ++j)
            lds_st<uint16_t>(lds, c_a2[i] + (j * 4 + s) * asub2, static_cast<uint16_t>(w[j]));
        }
        if (L >= 3) lds_st<float>(lds, c_ll[i], cf[0]);
      }
    }
    if (u + 1 < u_end) fetch(u + 1);
    WT_LDS_BARRIER();

    // ---- analysis levels 3..L from the raw LL of the level above (fp32 in LDS)
    levels_up<Geo, 3>(L, [&](auto lc) {
      const int l = lc;
      const int hl = pl.h[l], wl = pl.w[l], npos = pb * hl * wl;
      for (int idx = tid; idx < npos; idx += kMfmaBlock) {
        const int p = fast_div(idx, pl.mg_hw[l]);
        const int rem = idx - imul(p, hl * wl);
        const int i = fast_div(rem, pl.mg_w[l]);
        const int j = rem - imul(i, wl);
        const int hs = pl.h[l - 1], wsrc = pl.w[l - 1];
        const int so = pl.lloff[l - 1] + (imul(p, pl.llpl[l - 1]) + imul(2 * i, wsrc) + 2 * j) * 4;
        const bool r1 = 2 * i + 1 < hs, c1 = 2 * j + 1 < wsrc;
        const float a = lds_ld<float>(lds, so);
        const float b = c1 ? lds_ld<float>(lds, so + 4) : 0.f;
        const float cc = r1 ? lds_ld<float>(lds, so + wsrc * 4) : 0.f;
        const float d = (r1 && c1) ? lds_ld<float>(lds, so + wsrc * 4 + 4) : 0.f;
        const float s1 = a + b, d1 = a - b, s2 = cc + d, d2 = cc - d;
        const float cf[4] = {s1 + s2, s1 - s2, d1 + d2, d1 - d2};
        const int ao = pl.aoff[l] + (imul(imul(p, pl.prows[l]) + i + 2, pl.pitch[l]) + j + 2) * 2;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          uint32_t w[NS];
          split_pair<NS>(cf[s], 0.f, w);
#pragma unroll
          for (int js = 0; js < NS; ++js)
            lds_st<uint16_t>(lds, ao + (js * 4 + s) * pl.asub[l], static_cast<uint16_t>(w[js]));
        }
        if (l < L) lds_st<float>(lds, pl.lloff[l] + (imul(p, pl.llpl[l]) + imul(i, wl) + j) * 4, cf[0]);
      }
      WT_LDS_BARRIER();
    });

    // ---- stage 1: the last wave runs levels L..2 (conv + inverse Haar -> Z_l), the others the base
    // conv and, when every wave has at most one level-1 tile, the detail sub-bands of that tile
    const int base_waves = L >= 2 ? 3 : 4;
    // level-1 convolution of sub-band s of a tile into acc (resident or table fragments)
    auto conv1 = [&](const TileLane& tl, int s, Acc& acc) {
      Frag bt[NS], bb[NS];
      load_b<NS>(lds, tl.boff + s * asub1, 4 * asub1, 4 * pitchB1, bt, bb);
      if constexpr (RES) {
        mma_tile<NS>(ra1t[s], ra1b[s], bt, bb, acc);
      } else {
        Frag at[NS], ab[NS];
        load_a<NS>(lds, toff + (1 + s - pl.tfirst) * kFragEntries * 16, tsplit, ent_top, ent_bot, at, ab);
        mma_tile<NS>(at, ab, bt, bb, acc);
      }
    };
    const bool early = ntile1 <= 4 && L >= 2;   // every wave's single level-1 tile starts before the barrier
    TileLane tl1 = {};
    Acc acc1[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) acc1[s].v[0] = acc1[s].v[1] = acc1[s].v[2] = acc1[s].v[3] = 0.f;
    if (L >= 2 && wave == 3) {
      WT_WAVE_PRIORITY(3);        // the other waves wait for this chain at the barrier
      levels_down<Geo, 2>(L, [&](auto lc) {
        const int l = lc;
        const int ntile = pl.ntile[l];
        const int pitchB = pl.pitch[l] * 2, asub = pl.asub[l];
        const int zo_in = pl.zoff[l + 1], zp_in = pl.zpitch[l + 1], zpl_in = pl.zpl[l + 1];
        const int zo = pl.zoff[l], zp = pl.zpitch[l], zpl_o = pl.zpl[l], zrows = 4 * pl.nbr[l - 1];
        const int tab = toff + (1 + 4 * (l - 1) - pl.tfirst) * kFragEntries * 16;
#pragma unroll 1
        for (int t = 0; t < ntile; ++t) {
          const TileLane tl = tile_lane(lds, t, n, q, pl.tcs[l], pl.nrow[l], pl.nbc[l], pl.rtoff[l], pl.aoff[l], pitchB);
          Acc acc[4];
#pragma unroll
          for (int s = 0; s < 4; ++s) acc[s].v[0] = acc[s].v[1] = acc[s].v[2] = acc[s].v[3] = 0.f;
          if (l < L) {
            const float4 z = lds_ld<float4>(lds, zo_in + (imul(tl.p, zpl_in) + imul(4 * tl.bi + q, zp_in) + 4 * tl.tc) * 4);
            acc[0].v[0] = z.x; acc[0].v[1] = z.y; acc[0].v[2] = z.z; acc[0].v[3] = z.w;
          }
          if constexpr (NS == 1) {       // every LDS read of the tile is issued before the first MFMA
            Frag at[4][NS], ab[4][NS], bt[4][NS], bb[4][NS];
#pragma unroll
            for (int s = 0; s < 4; ++s) {
              load_b<NS>(lds, tl.boff + s * asub, 4 * asub, 4 * pitchB, bt[s], bb[s]);
              load_a<NS>(lds, tab + s * kFragEntries * 16, tsplit, ent_top, ent_bot, at[s], ab[s]);
            }
#pragma unroll
            for (int s = 0; s < 4; ++s) mma_tile<NS>(at[s], ab[s], bt[s], bb[s], acc[s]);
          } else {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
              Frag at[NS], ab[NS], bt[NS], bb[NS];
              load_b<NS>(lds, tl.boff + s * asub, 4 * asub, 4 * pitchB, bt, bb);
              load_a<NS>(lds, tab + s * kFragEntries * 16, tsplit, ent_top, ent_bot, at, ab);
              mma_tile<NS>(at, ab, bt, bb, acc[s]);
            }
          }
          float top[8], bot[8];
          synth_rows(acc, top, bot);
          const int y = 2 * (4 * tl.bi + q), xx = 8 * tl.tc;
          if (tl.valid) {
#pragma unroll
            for (int half = 0; half < 2; ++half) {
              if (xx + 4 * half < zp) {
                const int o = zo + (imul(tl.p, zpl_o) + imul(y, zp) + xx + 4 * half) * 4;
                float4 a, b;
                a.x = top[4 * half]; a.y = top[4 * half + 1]; a.z = top[4 * half + 2]; a.w = top[4 * half + 3];
                b.x = bot[4 * half]; b.y = bot[4 * half + 1]; b.z = bot[4 * half + 2]; b.w = bot[4 * half + 3];
                if (y < zrows) lds_st<float4>(lds, o, a);
                if (y + 1 < zrows) lds_st<float4>(lds, o + zp * 4, b);
              }
            }
          }
        }
        WT_WAVE_SYNC_DIVERGENT();
      });
      WT_WAVE_PRIORITY(0);
    }
    if (wave < base_waves) {
      // contiguous tile range per wave; with one plane per unit and one block-row per tile the lower
      // patch half of a tile is the upper half of the next one and is loaded once
      const int t0 = wave * ntile0 / base_waves, t1 = (wave + 1) * ntile0 / base_waves;
      const bool chain = pb == 1 && tcs0 == 4;
      Frag at[NS], ab[NS], bt[NS], bb[NS];
      if constexpr (!RES) load_a<NS>(lds, toff - pl.tfirst * kFragEntries * 16, tsplit, ent_top, ent_bot, at, ab);
      bool have_top = false;
#pragma unroll 1
      for (int t = t0; t < t1; ++t) {
        const TileLane tl = tile_lane(lds, t, n, q, tcs0, nrow0, nbc0, rtoff0, aoff0, pitchB0);
        if (chain && have_top) {
#pragma unroll
          for (int j = 0; j < NS; ++j) {
            bt[j] = bb[j];
            bb[j] = lds_frag8(lds, tl.boff + j * asub0 + 4 * pitchB0);
          }
        } else {
          load_b<NS>(lds, tl.boff, asub0, 4 * pitchB0, bt, bb);
        }
        have_top = true;
        Acc acc;
        acc.v[0] = acc.v[1] = acc.v[2] = acc.v[3] = bias;
        if constexpr (RES) mma_tile<NS>(ra0t, ra0b, bt, bb, acc);
        else mma_tile<NS>(at, ab, bt, bb, acc);
        if (tl.valid) {
          float4 a; a.x = acc.v[0]; a.y = acc.v[1]; a.z = acc.v[2]; a.w = acc.v[3];
          lds_st<float4>(lds, zoff1 + (imul(tl.p, zpl1) + imul(4 * tl.bi + q, zpitch1) + 4 * tl.tc) * 4, a);
        }
      }
    }
    // the detail sub-bands of this wave's level-1 tile: they need nothing of this stage (the coarse-chain wave
    // runs them after its chain, which is shorter than the base-conv share of the others)
    if (early && wave < ntile1) {
      tl1 = tile_lane(lds, wave, n, q, tcs1, nrow1, nbc1, rtoff1, aoff1, pitchB1);
#pragma unroll
      for (int s = 1; s < 4; ++s) conv1(tl1, s, acc1[s]);
    }
    WT_LDS_BARRIER();

    // ---- stage 2: level 1 (conv, inverse Haar), plus the base conv from Z_1, to HBM
    {
      T* obase = out + (static_cast<size_t>(b0) * C + c) * HW;
      bool first_store = true;
#pragma unroll 1
      for (int t = wave; t < ntile1; t += 4) {
        if (!early) {
          tl1 = tile_lane(lds, t, n, q, tcs1, nrow1, nbc1, rtoff1, aoff1, pitchB1);
#pragma unroll
          for (int s = 0; s < 4; ++s) acc1[s].v[0] = acc1[s].v[1] = acc1[s].v[2] = acc1[s].v[3] = 0.f;
        }
        const int y = 2 * (4 * tl1.bi + q), xx = 8 * tl1.tc;
        const bool store_ok = tl1.valid && tl1.p < np;
        // the base-conv part of this lane's 2 x 8 pixels, read ahead of the convolutions
        const int zbase = zoff1 + (imul(tl1.p, zpl1) + imul(y, zpitch1) + xx) * 4;
        float4 z1[2][2];
#pragma unroll
        for (int rr = 0; rr < 2; ++rr)
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            z1[rr][half].x = z1[rr][half].y = z1[rr][half].z = z1[rr][half].w = 0.f;
            if (store_ok && y + rr < H && xx + 4 * half < W)
              z1[rr][half] = lds_ld<float4>(lds, zbase + (rr * zpitch1 + 4 * half) * 4);
          }
        if (L >= 2) {
          const float4 z = lds_ld<float4>(lds, zoff2 + (imul(tl1.p, zpl2) + imul(4 * tl1.bi + q, zpitch2) + 4 * tl1.tc) * 4);
          acc1[0].v[0] = z.x; acc1[0].v[1] = z.y; acc1[0].v[2] = z.z; acc1[0].v[3] = z.w;
        }
        conv1(tl1, 0, acc1[0]);
        if (!early) {
#pragma unroll
          for (int s = 1; s < 4; ++s) conv1(tl1, s, acc1[s]);
        }
        float top[8], bot[8];
        synth_rows(acc1, top, bot);
        if (first_store) {
          // the prefetch of the next unit has had this tile's convolutions to land; waiting for it here, ahead of
          // the first store, lets the stores drain behind the next unit's work instead of being waited for at its commit
          WT_WAIT_VMEM();
          first_store = false;
        }
        if (store_ok) {
          T* dbase = obase + static_cast<size_t>(tl1.p) * C * HW + imul(y, W) + xx;
#pragma unroll
          for (int rr = 0; rr < 2; ++rr) {
            if (y + rr >= H) continue;
            float* vals = rr ? bot : top;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
              const int x0 = xx + 4 * half;
              if (x0 >= W) continue;
              const float4 z = z1[rr][half];
              const float r0 = vals[4 * half] + z.x, r1 = vals[4 * half + 1] + z.y;
              const float r2 = vals[4 * half + 2] + z.z, r3 = vals[4 * half + 3] + z.w;
              T* dst = dbase + rr * W + 4 * half;
              if constexpr (VEC) {
                if constexpr (sizeof(T) == 4) {
                  float4 o4; o4.x = r0; o4.y = r1; o4.z = r2; o4.w = r3;
                  *reinterpret_cast<float4*>(dst) = o4;
                } else {
                  uint2 o2; o2.x = pack_bf16x2(r0, r1); o2.y = pack_bf16x2(r2, r3);
                  *reinterpret_cast<uint2*>(dst) = o2;
                }
              } else if constexpr (sizeof(T) == 2) {
                if (x0 + 3 < W) {      // four columns inside the row: one (unaligned) 8-byte store
                  uint2 o2; o2.x = pack_bf16x2(r0, r1); o2.y = pack_bf16x2(r2, r3);
                  pix_store4u(dst, o2);
                } else {
                  const float r[4] = {r0, r1, r2, r3};
#pragma unroll
                  for (int e = 0; e < 4; ++e)
                    if (x0 + e < W) dst[e] = from_f32<T>(r[e]);
                }
              } else {
                const float r[4] = {r0, r1, r2, r3};
#pragma unroll
                for (int e = 0; e < 4; ++e)
                  if (x0 + e < W) dst[e] = from_f32<T>(r[e]);
              }
            }
          }
        }
      }
    }
    WT_LDS_BARRIER();
  }
}

}  // namespace wt
