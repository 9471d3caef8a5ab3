// Runs the WTConv kernels on the host through the same C ABI as the GPU library, using
// the emulation runtime (tests/emu/emu_runtime.h).  Test infrastructure only.
//
//   emu_driver <in.bin> <out.bin>
// in.bin : int32 header {dims, B, C, H, W, K, L, dtype, pdtype, has_bias}, then float32
//          arrays x, g, base_w, base_b (if has_bias), base_s, then per level w_l, s_l.
// out.bin: float32 arrays out, dx, dbase_w, dbase_b (if has_bias), dbase_s, per level dw_l, ds_l.
// dims == 0: in.bin holds B floats after the header; out.bin receives each after a round trip through the kernels'
//          float -> half -> float conversions.
// With dtype/pdtype = 1 the driver rounds the arrays to bfloat16 storage first, with 2 to IEEE half.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../include/wtconv_hip.h"
#include "../../wtconv_amd/csrc/common.h"      // only for the half conversions of the dims == 0 mode

static uint16_t to_bf16(float f) {
  uint32_t u; std::memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}
static float from_bf16(uint16_t v) { uint32_t u = static_cast<uint32_t>(v) << 16; float f; std::memcpy(&f, &u, 4); return f; }

// IEEE half by way of the value: nearest multiple of the half's spacing at that magnitude (ties to even)
static uint16_t to_f16(float f) {
  const uint16_t sign = std::signbit(f) ? 0x8000u : 0u;
  const double a = std::fabs(static_cast<double>(f));
  if (std::isnan(f)) return sign | 0x7e00u;
  if (a >= 65520.0) return sign | 0x7c00u;
  int e = a > 0 ? std::ilogb(a) : -14;
  if (e < -14) e = -14;
  const double q = std::nearbyint(std::ldexp(a, 10 - e));      // in units of 2^(e-10); default rounding is to even
  uint32_t m = static_cast<uint32_t>(q);
  uint32_t bits = (e == -14 && m < 1024u) ? m : ((static_cast<uint32_t>(e + 15) << 10) + (m - 1024u));
  return static_cast<uint16_t>(sign | bits);
}
static float from_f16(uint16_t h) {
  const int ex = (h >> 10) & 31, man = h & 1023;
  double v = ex == 31 ? (man ? NAN : INFINITY) : ex == 0 ? std::ldexp(man, -24) : std::ldexp(1024 + man, ex - 25);
  return static_cast<float>((h & 0x8000u) ? -v : v);
}

struct Buf {
  std::vector<float> f;       // float view (input as read / output to write)
  std::vector<uint16_t> h;    // bf16 storage when dtype == 1, half storage when dtype == 2
  int dtype = 0;
  void* ptr() { return dtype ? static_cast<void*>(h.data()) : static_cast<void*>(f.data()); }
  void pack() {
    if (dtype) { h.resize(f.size()); for (size_t i = 0; i < f.size(); ++i) h[i] = dtype == 2 ? to_f16(f[i]) : to_bf16(f[i]); }
  }
  void unpack() { if (dtype) for (size_t i = 0; i < f.size(); ++i) f[i] = dtype == 2 ? from_f16(h[i]) : from_bf16(h[i]); }
};

static Buf read_buf(FILE* fp, size_t n, int dtype) {
  Buf b; b.dtype = dtype; b.f.resize(n);
  if (n && fread(b.f.data(), 4, n, fp) != n) { fprintf(stderr, "short read\n"); exit(2); }
  b.pack();
  return b;
}
static Buf out_buf(size_t n, int dtype) { Buf b; b.dtype = dtype; b.f.assign(n, -777.f); b.pack(); return b; }

int main(int argc, char** argv) {
  if (argc != 3) { fprintf(stderr, "usage: emu_driver in.bin out.bin\n"); return 2; }
  FILE* fp = fopen(argv[1], "rb");
  if (!fp) { perror("open"); return 2; }
  int32_t hd[10];
  if (fread(hd, 4, 10, fp) != 10) return 2;
  const int dims = hd[0], B = hd[1], C = hd[2], H = hd[3], W = hd[4], K = hd[5], L = hd[6];
  const int dtype = hd[7], pdtype = hd[8], has_bias = hd[9];
  if (dims == 0) {
    std::vector<float> v(B);
    if (B && fread(v.data(), 4, v.size(), fp) != v.size()) return 2;
    fclose(fp);
    for (float& f : v) f = wt::f16_bits_to_f32(wt::f32_to_f16_bits(f));
    FILE* fo = fopen(argv[2], "wb");
    if (!fo) { perror("open"); return 2; }
    fwrite(v.data(), 4, v.size(), fo);
    fclose(fo);
    return 0;
  }
  if (dims == 3 || dims == 4) {
    // block passes: header {dims, B, C, H, W, nhwc (K slot), unused, dtype, pdtype, unused}
    //   dims == 3: in x, dy, weight, bias            -> out, dx, dweight, dbias       (channel norm, forward + backward)
    //   dims == 4: in y (NHWC), shortcut, gamma, dout -> out, dy (NHWC), dgamma        (block residual, forward + backward)
    const int HW = H * W, nhwc = K;
    const size_t P = static_cast<size_t>(B) * C * HW;
    Buf a0 = read_buf(fp, P, dtype), a1 = read_buf(fp, P, dtype);
    Buf p0 = read_buf(fp, C, pdtype);
    Buf p1 = dims == 3 ? read_buf(fp, C, pdtype) : read_buf(fp, P, dtype);
    fclose(fp);
    Buf o0 = out_buf(P, dtype), o1 = out_buf(P, dtype);
    std::vector<float> g0(C, -777.f), g1(C, -777.f);
    std::vector<char> ws(wtconv_block_workspace_bytes(B, C, HW, dtype));
    int rc;
    if (dims == 3) {
      rc = wtconv_channel_norm(a0.ptr(), o0.ptr(), p0.ptr(), p1.ptr(), B, C, HW, 1e-6f, dtype, pdtype, nhwc, nullptr);
      if (rc) { fprintf(stderr, "channel_norm: %s\n", wtconv_last_error()); return 3; }
      rc = wtconv_channel_norm_backward(a0.ptr(), a1.ptr(), p0.ptr(), o1.ptr(), g0.data(), g1.data(), B, C, HW, 1e-6f, dtype,
                                        pdtype, nhwc, ws.data(), ws.size(), nullptr);
      if (rc) { fprintf(stderr, "channel_norm_backward: %s\n", wtconv_last_error()); return 3; }
    } else {
      rc = wtconv_block_residual(a0.ptr(), a1.ptr(), p0.ptr(), o0.ptr(), B, C, HW, dtype, pdtype, nullptr);
      if (rc) { fprintf(stderr, "block_residual: %s\n", wtconv_last_error()); return 3; }
      rc = wtconv_block_residual_backward(p1.ptr(), a0.ptr(), p0.ptr(), o1.ptr(), g0.data(), B, C, HW, dtype, pdtype,
                                          ws.data(), ws.size(), nullptr);
      if (rc) { fprintf(stderr, "block_residual_backward: %s\n", wtconv_last_error()); return 3; }
    }
    o0.unpack(); o1.unpack();
    FILE* fo = fopen(argv[2], "wb");
    if (!fo) { perror("open out"); return 2; }
    fwrite(o0.f.data(), 4, P, fo);
    fwrite(o1.f.data(), 4, P, fo);
    fwrite(g0.data(), 4, C, fo);
    if (dims == 3) fwrite(g1.data(), 4, C, fo);
    fclose(fo);
    return 0;
  }
  const int S = dims == 2 ? 4 : 2;
  const size_t KK = dims == 2 ? static_cast<size_t>(K) * K : K;
  const size_t P = static_cast<size_t>(B) * C * H * W;   // 1-D: H == 1, W == N
  Buf x = read_buf(fp, P, dtype), g = read_buf(fp, P, dtype);
  Buf bw = read_buf(fp, C * KK, pdtype);
  Buf bb = read_buf(fp, has_bias ? C : 0, pdtype);
  Buf bs = read_buf(fp, C, pdtype);
  std::vector<Buf> ws, ss;
  for (int l = 0; l < L; ++l) { ws.push_back(read_buf(fp, S * C * KK, pdtype)); ss.push_back(read_buf(fp, S * C, pdtype)); }
  fclose(fp);

  wtconv_params prm = {};
  prm.base_weight = bw.ptr(); prm.base_bias = has_bias ? bb.ptr() : nullptr; prm.base_scale = bs.ptr();
  for (int l = 0; l < L; ++l) { prm.wt_weight[l] = ws[l].ptr(); prm.wt_scale[l] = ss[l].ptr(); }

  Buf out = out_buf(P, dtype), dx = out_buf(P, dtype);
  std::vector<float> dbw(C * KK, -777.f), dbb(C, -777.f), dbs(C, -777.f);
  std::vector<std::vector<float>> dws(L, std::vector<float>(S * C * KK, -777.f)), dss(L, std::vector<float>(S * C, -777.f));
  wtconv_param_grads gr = {};
  gr.base_weight = dbw.data(); gr.base_bias = has_bias ? dbb.data() : nullptr; gr.base_scale = dbs.data();
  for (int l = 0; l < L; ++l) { gr.wt_weight[l] = dws[l].data(); gr.wt_scale[l] = dss[l].data(); }

  int rc = 0;
  const char* fused_env = getenv("WT_EMU_FUSED_BWD");      // "1": the whole backward pass through wtconv*_backward
  const bool fused = fused_env != nullptr && fused_env[0] == '1';
  auto ws_alloc = [&](size_t bytes) { return std::vector<char>(bytes); };   // exact size: ASan guards it
  if (dims == 2) {
    auto w0 = ws_alloc(wtconv2d_workspace_bytes(B, C, H, W, K, L, WTCONV_PASS_FORWARD));
    rc = wtconv2d_forward(x.ptr(), out.ptr(), &prm, B, C, H, W, K, L, dtype, pdtype, w0.data(), w0.size(), nullptr);
    if (rc) { fprintf(stderr, "forward: %s\n", wtconv_last_error()); return 3; }
    if (fused) {
      auto w3 = ws_alloc(wtconv2d_workspace_bytes(B, C, H, W, K, L, WTCONV_PASS_BACKWARD));
      rc = wtconv2d_backward(x.ptr(), g.ptr(), dx.ptr(), &prm, &gr, B, C, H, W, K, L, dtype, pdtype, w3.data(), w3.size(), nullptr);
      if (rc) { fprintf(stderr, "backward: %s\n", wtconv_last_error()); return 3; }
    } else {
    auto w1 = ws_alloc(wtconv2d_workspace_bytes(B, C, H, W, K, L, WTCONV_PASS_BACKWARD_INPUT));
    rc = wtconv2d_backward_input(g.ptr(), dx.ptr(), &prm, B, C, H, W, K, L, dtype, pdtype, w1.data(), w1.size(), nullptr);
    if (rc) { fprintf(stderr, "backward_input: %s\n", wtconv_last_error()); return 3; }
    auto w2 = ws_alloc(wtconv2d_workspace_bytes(B, C, H, W, K, L, WTCONV_PASS_BACKWARD_PARAMS));
    rc = wtconv2d_backward_params(x.ptr(), g.ptr(), &prm, &gr, B, C, H, W, K, L, dtype, pdtype, w2.data(), w2.size(), nullptr);
    if (rc) { fprintf(stderr, "backward_params: %s\n", wtconv_last_error()); return 3; }
    }
  } else {
    const int N = W;
    auto w0 = ws_alloc(wtconv1d_workspace_bytes(B, C, N, K, L, WTCONV_PASS_FORWARD));
    rc = wtconv1d_forward(x.ptr(), out.ptr(), &prm, B, C, N, K, L, dtype, pdtype, w0.data(), w0.size(), nullptr);
    if (rc) { fprintf(stderr, "forward: %s\n", wtconv_last_error()); return 3; }
    if (fused) {
      auto w3 = ws_alloc(wtconv1d_workspace_bytes(B, C, N, K, L, WTCONV_PASS_BACKWARD));
      rc = wtconv1d_backward(x.ptr(), g.ptr(), dx.ptr(), &prm, &gr, B, C, N, K, L, dtype, pdtype, w3.data(), w3.size(), nullptr);
      if (rc) { fprintf(stderr, "backward: %s\n", wtconv_last_error()); return 3; }
    } else {
    auto w1 = ws_alloc(wtconv1d_workspace_bytes(B, C, N, K, L, WTCONV_PASS_BACKWARD_INPUT));
    rc = wtconv1d_backward_input(g.ptr(), dx.ptr(), &prm, B, C, N, K, L, dtype, pdtype, w1.data(), w1.size(), nullptr);
    if (rc) { fprintf(stderr, "backward_input: %s\n", wtconv_last_error()); return 3; }
    auto w2 = ws_alloc(wtconv1d_workspace_bytes(B, C, N, K, L, WTCONV_PASS_BACKWARD_PARAMS));
    rc = wtconv1d_backward_params(x.ptr(), g.ptr(), &prm, &gr, B, C, N, K, L, dtype, pdtype, w2.data(), w2.size(), nullptr);
    if (rc) { fprintf(stderr, "backward_params: %s\n", wtconv_last_error()); return 3; }
    }
  }
  out.unpack(); dx.unpack();
  FILE* fo = fopen(argv[2], "wb");
  if (!fo) { perror("open out"); return 2; }
  fwrite(out.f.data(), 4, P, fo);
  fwrite(dx.f.data(), 4, P, fo);
  fwrite(dbw.data(), 4, dbw.size(), fo);
  if (has_bias) fwrite(dbb.data(), 4, dbb.size(), fo);
  fwrite(dbs.data(), 4, dbs.size(), fo);
  for (int l = 0; l < L; ++l) { fwrite(dws[l].data(), 4, dws[l].size(), fo); fwrite(dss[l].data(), 4, dss[l].size(), fo); }
  fclose(fo);
  return 0;
}
