// Geometry shared by the convolution kernels.
#pragma once

#include "mcn_internal.hpp"

namespace mcn {

struct ConvP {
  int H, W, C, N;
  int FH, FW, FC, K;
  int sy, sx, pt, pl, dy, dx;
  int outH, outW;
  int groups, Kg;  // Kg = filters per group
};

// Validates like the MEX driver (vl_nnconv.cu:269-342) and fills the derived fields.
int conv_setup(const mcn_conv_geom* g, const char* who, ConvP* p);

// direct (one accumulator per output element) kernels: any stride / dilation / padding / groups
int conv_forward_direct(hipStream_t s, const ConvP& p, float* y, float outMult, const float* x, float inMult,
                        const float* f, const float* b);
int conv_backward_data_direct(hipStream_t s, const ConvP& p, float* dx, const float* f, const float* dy);
int conv_backward_filter_direct(hipStream_t s, const ConvP& p, float* df, const float* x, const float* dy);

// MFMA implicit-GEMM kernels (groups == 1).  *_supported says whether the fast path covers `p`.
bool conv_mfma_forward_supported(const ConvP& p);
bool conv_mfma_backward_data_supported(const ConvP& p);
bool conv_mfma_backward_filter_supported(const ConvP& p);
size_t conv_mfma_workspace_bytes(const ConvP& p, int product);
int conv_forward_mfma(hipStream_t s, const ConvP& p, float* y, float outMult, const float* x, float inMult,
                      const float* f, const float* b, void* ws, size_t wsBytes);
int conv_backward_data_mfma(hipStream_t s, const ConvP& p, float* dx, const float* f, const float* dy, void* ws,
                            size_t wsBytes);
int conv_backward_filter_mfma(hipStream_t s, const ConvP& p, float* df, const float* x, const float* dy, void* ws,
                              size_t wsBytes);

// Parameters of the pixel-major products (forward / backward-data): out[co, m] = sum_R wt[R][co] * in[ci(R), pixel(m) + tap(R)]
struct PixP {
  int IH, IW, Cin;    // grid and channels of the gathered tensor
  int OH, OW, Cout;   // grid and channels of the produced tensor
  int N;
  int FH, T;          // filter height, taps = FH*FW
  int sy, sx;         // gathered row = oh*sy + dh(tap)
  int dhBase, dhStep, dwBase, dwStep;
  int R;              // reduction length = T*Cin
  int coutPad;        // row pitch of wt
  int M;              // OH*OW*N (< 2^31)
  float alpha, beta;
  FastDiv byQ, byOH, byT;  // Q = OH*OW; T = taps
  int advC, advT;          // 16 = advC*T + advT (reduction rows per step)
};

// Weights-stationary variant (conv_ws.hip) for filter banks that fit in LDS: wt is the packed bank in tap-major
// order (R = ci + Cin*t).  Sets *handled when it took the work.
int conv_ws_launch(hipStream_t s, const char* who, float* out, const float* in, const float* wt, const float* bias,
                   const PixP& p, int* handled);

}  // namespace mcn
