// Patch matrix of a 2-D convolution and its transpose: the out-channel-sharded convolution runs as the column-sharded
// product  Y[N*Ho*Wo, Co] = patches[N*Ho*Wo, Ci*kh*kw] x W^T  on the GEMM kernel (a shard's weight [Co_s, Ci, kh, kw]
// is, as stored, the row-major [Co_s, Ci*kh*kw] operand), with the input gradient folded back from the patch gradients.
#include "common.h"

#include "rtp_hip.h"

namespace rtp {

struct ConvGeom {
  long n, c, h, w, kh, kw, sh, sw, ph, pw, dh, dw, ho, wo;
};

// patches[(n*Ho + ho)*Wo + wo][(ci*kh + i)*kw + j] = x[n][ci][ho*sh - ph + i*dh][wo*sw - pw + j*dw] (0 outside);
// columns K .. ld-1 of a padded row pitch are zero-filled.  One thread per element, consecutive threads along a row.
template <typename T>
__global__ __launch_bounds__(256) void im2col_kernel(const T* x, long sx_n, long sx_c, long sx_h, long sx_w, ConvGeom g,
                                                     T* cols, long ld) {
  const long total = g.n * g.ho * g.wo * ld;
  const long K = g.c * g.kh * g.kw;
  const long stride = (long)gridDim.x * blockDim.x;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
    const long k = idx % ld, row = idx / ld;
    T v = from_f32<T>(0.0f);
    if (k < K) {
      const long j = k % g.kw, i = (k / g.kw) % g.kh, ci = k / (g.kw * g.kh);
      const long wo = row % g.wo, ho = (row / g.wo) % g.ho, n = row / (g.wo * g.ho);
      const long h = ho * g.sh - g.ph + i * g.dh, w = wo * g.sw - g.pw + j * g.dw;
      if (h >= 0 && h < g.h && w >= 0 && w < g.w) v = x[n * sx_n + ci * sx_c + h * sx_h + w * sx_w];
    }
    cols[idx] = v;
  }
}

// dx[n][ci][h][w] = sum over (i, j) with h = ho*sh - ph + i*dh, w = wo*sw - pw + j*dw of
// dpatches[(n*Ho + ho)*Wo + wo][(ci*kh + i)*kw + j]: a gather per input element, fp32 sum in ascending (i, j), no atomics.
template <typename T>
__global__ __launch_bounds__(256) void col2im_kernel(const T* dcols, long ld, ConvGeom g, T* dx) {
  const long total = g.n * g.c * g.h * g.w;
  const long stride = (long)gridDim.x * blockDim.x;
  for (long idx = (long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
    const long w = idx % g.w, h = (idx / g.w) % g.h, ci = (idx / (g.w * g.h)) % g.c, n = idx / (g.w * g.h * g.c);
    float acc = 0.0f;
    for (long i = 0; i < g.kh; ++i) {
      const long hn = h + g.ph - i * g.dh;
      if (hn < 0 || hn % g.sh != 0) continue;
      const long ho = hn / g.sh;
      if (ho >= g.ho) continue;
      for (long j = 0; j < g.kw; ++j) {
        const long wn = w + g.pw - j * g.dw;
        if (wn < 0 || wn % g.sw != 0) continue;
        const long wo = wn / g.sw;
        if (wo >= g.wo) continue;
        acc += to_f32(dcols[((n * g.ho + ho) * g.wo + wo) * ld + (ci * g.kh + i) * g.kw + j]);
      }
    }
    dx[idx] = from_f32<T>(acc);
  }
}

static int check_geom(const char* who, const rtp_conv_geom* geom, ConvGeom& g) {
  RTP_REQUIRE(geom, "%s: null geometry", who);
  g = ConvGeom{geom->n, geom->c, geom->h, geom->w, geom->kh, geom->kw, geom->sh, geom->sw,
               geom->ph, geom->pw, geom->dh, geom->dw, geom->ho, geom->wo};
  RTP_REQUIRE(g.n >= 1 && g.c >= 1 && g.h >= 1 && g.w >= 1 && g.kh >= 1 && g.kw >= 1, "%s: sizes must be >= 1", who);
  RTP_REQUIRE(g.sh >= 1 && g.sw >= 1 && g.dh >= 1 && g.dw >= 1 && g.ph >= 0 && g.pw >= 0,
              "%s: stride and dilation must be >= 1, padding >= 0", who);
  const long span_h = g.h + 2 * g.ph - g.dh * (g.kh - 1) - 1, span_w = g.w + 2 * g.pw - g.dw * (g.kw - 1) - 1;
  RTP_REQUIRE(span_h >= 0 && span_w >= 0, "%s: kernel larger than the padded input", who);
  RTP_REQUIRE(g.ho == span_h / g.sh + 1 && g.wo == span_w / g.sw + 1,
              "%s: output size %lld x %lld does not match the geometry (expected %lld x %lld)", who, (long long)g.ho,
              (long long)g.wo, (long long)(span_h / g.sh + 1), (long long)(span_w / g.sw + 1));
  return RTP_OK;
}

static unsigned flat_grid(long total) { return (unsigned)std::min<long>(16384, std::max<long>(1, ceil_div(total, 256))); }

}  // namespace rtp

using namespace rtp;

extern "C" int rtp_im2col(void* stream, int dtype, const void* x, int64_t sx_n, int64_t sx_c, int64_t sx_h,
                          int64_t sx_w, const rtp_conv_geom* geom, void* cols, int64_t ld_cols) {
  ConvGeom g;
  if (int rc = check_geom("rtp_im2col", geom, g)) return rc;
  RTP_REQUIRE(x && cols, "rtp_im2col: null pointer");
  RTP_REQUIRE(dtype == RTP_F32 || dtype == RTP_BF16, "rtp_im2col: unknown dtype %d", dtype);
  RTP_REQUIRE(ld_cols >= g.c * g.kh * g.kw, "rtp_im2col: row pitch %lld below the patch length %lld",
              (long long)ld_cols, (long long)(g.c * g.kh * g.kw));
  hipStream_t st = (hipStream_t)stream;
  const long total = g.n * g.ho * g.wo * ld_cols;
  const double esz = dtype == RTP_F32 ? 4.0 : 2.0;
  ProfileScope prof(st, "im2col", 0.0, esz * ((double)total + (double)g.n * g.c * g.h * g.w));
  if (dtype == RTP_F32)
    hipLaunchKernelGGL(im2col_kernel<float>, dim3(flat_grid(total)), dim3(256), 0, st, (const float*)x, (long)sx_n,
                       (long)sx_c, (long)sx_h, (long)sx_w, g, (float*)cols, (long)ld_cols);
  else
    hipLaunchKernelGGL(im2col_kernel<bf16_t>, dim3(flat_grid(total)), dim3(256), 0, st, (const bf16_t*)x, (long)sx_n,
                       (long)sx_c, (long)sx_h, (long)sx_w, g, (bf16_t*)cols, (long)ld_cols);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" int rtp_col2im(void* stream, int dtype, const void* dcols, int64_t ld_dcols, const rtp_conv_geom* geom,
                          void* dx) {
  ConvGeom g;
  if (int rc = check_geom("rtp_col2im", geom, g)) return rc;
  RTP_REQUIRE(dcols && dx, "rtp_col2im: null pointer");
  RTP_REQUIRE(dtype == RTP_F32 || dtype == RTP_BF16, "rtp_col2im: unknown dtype %d", dtype);
  RTP_REQUIRE(ld_dcols >= g.c * g.kh * g.kw, "rtp_col2im: row pitch %lld below the patch length %lld",
              (long long)ld_dcols, (long long)(g.c * g.kh * g.kw));
  hipStream_t st = (hipStream_t)stream;
  const long total = g.n * g.c * g.h * g.w;
  const double esz = dtype == RTP_F32 ? 4.0 : 2.0;
  ProfileScope prof(st, "col2im", 0.0, esz * ((double)total + (double)g.n * g.ho * g.wo * g.c * g.kh * g.kw));
  if (dtype == RTP_F32)
    hipLaunchKernelGGL(col2im_kernel<float>, dim3(flat_grid(total)), dim3(256), 0, st, (const float*)dcols,
                       (long)ld_dcols, g, (float*)dx);
  else
    hipLaunchKernelGGL(col2im_kernel<bf16_t>, dim3(flat_grid(total)), dim3(256), 0, st, (const bf16_t*)dcols,
                       (long)ld_dcols, g, (bf16_t*)dx);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}
