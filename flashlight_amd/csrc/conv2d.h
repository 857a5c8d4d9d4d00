// Internal interface between the convolution entry points and their kernels.
#pragma once
#include "common.h"

namespace flhip {

struct ConvGeom {
  int N, C, H, W, K, KH, KW, OH, OW;
  int sy, sx, py, px, dly, dlx, groups;
  int Cg, Kg;  // channels per group
};

// Implicit-GEMM MFMA kernels (conv2d_mfma.hip).  Each returns FLHIP_OK after
// enqueueing, or -1 when the shape is outside what the kernel handles (the
// caller then uses the direct kernels).
int mfma_conv_fwd(const ConvGeom& g, int dtype, const void* x, const void* w, const float* bias,
                  void* y, hipStream_t s);
int mfma_conv_bwd_data(const ConvGeom& g, int dtype, const void* dy, const void* w, void* dx,
                       hipStream_t s);
int mfma_conv_bwd_filter(const ConvGeom& g, int dtype, const void* x, const void* dy, float* dw,
                         float* db, void* ws, size_t ws_bytes, hipStream_t s);
size_t mfma_conv_bwd_filter_ws(const ConvGeom& g, int dtype);

// LDS-resident-slab kernels for stride-1 convolutions with small windows
// (conv2d_mfma_slab.hip); same return convention.
int mfma_slab_conv_fwd(const ConvGeom& g, int dtype, const void* x, const void* w,
                       const float* bias, void* y, hipStream_t s);
int mfma_slab_wgrad(const ConvGeom& g, int dtype, const void* x, const void* dy, float* dw,
                    float* db, void* ws, size_t ws_bytes, hipStream_t s);
size_t mfma_slab_wgrad_ws(const ConvGeom& g, int dtype);
bool mfma_slab_wgrad_applies(const ConvGeom& g);
int mfma_slab_conv_bwd_data(const ConvGeom& g, int dtype, const void* dy, const void* w, void* dx,
                            hipStream_t s);

// 1x1 convolutions without padding as GEMMs (conv2d_mfma_pointwise.hip); same return
// convention.
int mfma_pointwise_conv_fwd(const ConvGeom& g, int dtype, const void* x, const void* w,
                            const float* bias, void* y, hipStream_t s, int ksplit = 1);
int mfma_pointwise_conv_bwd_data(const ConvGeom& g, int dtype, const void* dy, const void* w,
                                 void* dx, hipStream_t s, const float* bias = nullptr, int ksplit = 1);
// bf16 storage on the bf16 matrix cores: 1x1 windows without padding over planes of at
// least 4 positions, channel counts multiples of 8; -1 otherwise.  Strided windows need
// mfma_pointwise16_lattice_ws() bytes of workspace (the input's lattice points / the compact
// gradient) and return -1 without it; so do the backward passes of strided windows with 2 to 9
// taps, which gather the taps next to the channels (bwd = true in the query).
int mfma_pointwise16_conv_fwd(const ConvGeom& g, const void* x, const void* w, const float* bias, void* y,
                              hipStream_t s, void* ws, size_t ws_bytes, int dtype);
int mfma_pointwise16_conv_bwd_data_add(const ConvGeom& g, const void* dy, const void* w, const void* addend, void* dx,
                                       hipStream_t s, int dtype);
int mfma_pointwise16_conv_bwd_data(const ConvGeom& g, const void* dy, const void* w, void* dx, hipStream_t s,
                                   void* ws, size_t ws_bytes, int dtype);
size_t mfma_pointwise16_lattice_ws(const ConvGeom& g, bool bwd);
size_t mfma_pointwise16_wgrad_ws(const ConvGeom& g);
int mfma_pointwise16_wgrad(const ConvGeom& g, const void* x, const void* dy, float* dw, float* db, void* ws,
                           size_t ws_bytes, hipStream_t s, const void* gathered, int dtype);
// bytes of gathered input that the forward pass leaves at the start of its workspace for the filter gradient (0: none)
size_t mfma_pointwise16_gathered_bytes(const ConvGeom& g);
// fp32, stride 1, few tiles and a long contraction: the contraction in slices through
// mfma_pointwise_split_ws() bytes of workspace; -1 when it does not apply or the room is missing
size_t mfma_pointwise_split_ws(const ConvGeom& g, int dtype, bool bwd);
int mfma_pointwise_conv_split(const ConvGeom& g, int dtype, bool bwd, const void* src, const void* w,
                              const float* bias, void* dst, void* ws, size_t ws_bytes, hipStream_t s);
// column-major C = op(A) op(B) on the 1x1 kernels (mode 0: A B, 1: A^T B, 2: A B^T);
// -1 when it does not apply
int mfma_gemm(int dtype, int mode, const void* A, const void* B, void* C, int M, int N, int K,
              const float* bias_rows, hipStream_t s, int ksplit = 1);
int mfma_gemm_slices(int K, int ksplit);
int mfma_gemm_planes(int mode, const void* A, const void* B, void* C, int M, int N, int K, const float* bias_rows,
                     hipStream_t s);
// the same three products in 16-bit storage on the 16-bit matrix instructions (conv2d_mfma_pointwise_dma_bf16.hip)
int mfma_gemm16(int dtype, int mode, const void* A, const void* B, void* C, int M, int N, int K,
                const float* bias_rows, hipStream_t s, void* ws, size_t ws_bytes);
size_t mfma_gemm16_ws_bytes(int dtype, int mode, int M, int N, int K);
// column-major C = A * B^T on a kernel of its own (both operands contiguous along the
// surviving dimension); slices > 1 (f32): partial products M * N floats apart
int gemm_nt(int dtype, const void* A, const void* B, void* C, int M, int N, int K, int slices, hipStream_t s);
// windows with several taps on the same tile machinery, any stride / padding / dilation
int mfma_tapped_conv_fwd(const ConvGeom& g, int dtype, const void* x, const void* w,
                         const float* bias, void* y, hipStream_t s, void* ws = nullptr, size_t ws_bytes = 0);
int mfma_tapped_conv_bwd_data(const ConvGeom& g, int dtype, const void* dy, const void* w,
                              void* dx, hipStream_t s, void* ws = nullptr, size_t ws_bytes = 0);
// with that many bytes of workspace the weights are reordered so that a tap's tile is contiguous
size_t mfma_tapped_ws(const ConvGeom& g, int dtype, bool bwd);
size_t mfma_pointwise_wgrad_ws(const ConvGeom& g);
// windows = false: only 1x1 without padding; true: any window, one tap per workgroup
int mfma_pointwise_wgrad(const ConvGeom& g, int dtype, const void* x, const void* dy, float* dw,
                         float* db, void* ws, size_t ws_bytes, bool windows, hipStream_t s,
                         int max_slices = 0);

// Adds the slices of a split filter gradient in a fixed order (conv2d_mfma_wgrad.hip):
// slice s holds E floats of dw followed by K floats of db at part + s * (E + K).
void wgrad_reduce_launch(const float* part, int nsplit, int E, int K, int want_db, float* dw,
                         float* db, hipStream_t s);

// bf16-storage variants on the bf16 matrix cores (conv2d_mfma_slab_bf16.hip,
// conv2d_mfma_wgrad_slab_bf16.hip); same return convention.
// bf16 forward of a first layer: few input channels, window rows of at most 8 columns, even column stride
// (conv2d_mfma_first_bf16.hip)
int mfma_first16_conv_fwd(const ConvGeom& g, const void* x, const void* w, const float* bias, void* y,
                          hipStream_t s, int dtype);
size_t mfma_first16_wgrad_ws(const ConvGeom& g);
int mfma_first16_wgrad(const ConvGeom& g, const void* x, const void* dy, float* dw, float* db, void* ws,
                       size_t ws_bytes, hipStream_t s, int dtype);
// backward-data of a stride-2 window over at most 4 input channels (the stem), any storage type, as a 4 x 4
// stride-1 window over the output gradient onto the 2 x 2 cells of the input gradient (conv2d_mfma_cells.hip)
int mfma_cells_conv_bwd_data(const ConvGeom& g, int dtype, const void* dy, const void* w, void* dx, hipStream_t s);
// the forward pass of the same layers on the same cells (the window spans at most 4 x 4 cells of the input)
int mfma_cells_conv_fwd(const ConvGeom& g, int dtype, const void* x, const void* w, const float* bias, void* y, hipStream_t s);
// bf16 3x3 stride-1 pad-1 over 64 source channels, whole contraction per workgroup (conv2d_mfma_strip_bf16.hip)
// bf16 1x1 stride-1 convolutions with operand tiles copied to LDS by the loads themselves
// (conv2d_mfma_pointwise_dma_bf16.hip); -1 when the shape is not theirs.  addend (or null): added
// to the rounded input gradient.
int mfma_pwd16_conv_fwd(const ConvGeom& g, const void* x, const void* w, const float* bias, void* y, hipStream_t s,
                        int dtype = FLHIP_BF16);
int mfma_pwd16_conv_bwd_data(const ConvGeom& g, const void* dy, const void* w, const void* addend, void* dx,
                             hipStream_t s, int dtype);
// their filter gradient (no bias gradient; at least 128 channels on both sides); partial tiles in ws
size_t mfma_pwd16_wgrad_ws(const ConvGeom& g);
// workgroups the bf16 slab kernel's forward pass would launch (0: not its shape)
long long mfma_slab16_conv_fwd_workgroups(const ConvGeom& g);
int mfma_pwd16_wgrad(const ConvGeom& g, const void* x, const void* dy, float* dw, void* ws, size_t ws_bytes, hipStream_t s,
                     int dtype = FLHIP_BF16);
int mfma_strip16_conv_fwd(const ConvGeom& g, const void* x, const void* w, const float* bias, void* y,
                          hipStream_t s, int dtype);
int mfma_strip16_conv_bwd_data(const ConvGeom& g, const void* dy, const void* w, void* dx, hipStream_t s, int dtype);
int mfma_slab16_conv_fwd(const ConvGeom& g, const void* x, const void* w, const float* bias, void* y,
                         hipStream_t s, int dtype);
int mfma_slab16_conv_bwd_data(const ConvGeom& g, const void* dy, const void* w, void* dx,
                              hipStream_t s, int dtype);
// windows of one row (KH = 1, 2 to 32 taps, column stride 1 or 2, no groups, 16 to 256 contraction channels) in bf16
// or fp32 storage through channels-last rows and fragment-ordered weights in mfma_tap1d_conv_ws() bytes of workspace
// (conv2d_mfma_tap1d.hip); -1 when the shape is not theirs or the room is missing
size_t mfma_tap1d_conv_ws(const ConvGeom& g, int dtype, bool bwd);
int mfma_tap1d_conv_fwd(const ConvGeom& g, int dtype, const void* x, const void* w, const float* bias, void* y, hipStream_t s,
                        void* ws, size_t ws_bytes);
int mfma_tap1d_conv_bwd_data(const ConvGeom& g, int dtype, const void* dy, const void* w, void* dx, hipStream_t s, void* ws,
                             size_t ws_bytes);
// 3x3 windows of stride 1 and padding 1 over small planes on the same kernels: every plane of the batch in one
// sequence (rows followed by a zero column, planes separated by a zero row), 65 to 512 (fp32: 256) contraction channels;
// operands in mfma_tap2d_conv_ws() bytes of workspace; -1 when the shape is not theirs or the room is missing
size_t mfma_tap2d_conv_ws(const ConvGeom& g, int dtype, bool bwd);
int mfma_tap2d_conv_fwd(const ConvGeom& g, int dtype, const void* x, const void* w, const float* bias, void* y, hipStream_t s,
                        void* ws, size_t ws_bytes);
int mfma_tap2d_conv_bwd_data(const ConvGeom& g, int dtype, const void* dy, const void* w, void* dx, hipStream_t s, void* ws,
                             size_t ws_bytes);
// their filter gradient (6 to 23 taps; bf16: an even number of result positions per row): the channels-last rows and
// the workgroups' tiles in mfma_tap1d_wgrad_ws() bytes of workspace
size_t mfma_tap1d_wgrad_ws(const ConvGeom& g, int dtype);
int mfma_tap1d_wgrad(const ConvGeom& g, int dtype, const void* x, const void* dy, float* dw, float* db, void* ws,
                     size_t ws_bytes, hipStream_t s, const void* rows = nullptr);
// bytes of channels-last rows that their forward pass leaves at the start of its workspace and the filter gradient
// takes as `rows` in place of x (0: the two passes do not both apply)
size_t mfma_tap1d_rows_bytes(const ConvGeom& g, int dtype);
// 3x3 filter gradient with operand rows copied straight to LDS (conv2d_mfma_wgrad_dma_bf16.hip)
size_t mfma_wgrad_dma16_ws(const ConvGeom& g);
// tile: 0 = by the measured rule, 32 / 64 = that tile side or decline
int mfma_wgrad_dma16(const ConvGeom& g, const void* x, const void* dy, float* dw, float* db, void* ws, size_t ws_bytes,
                     hipStream_t s, int tile, int dtype);
size_t mfma_wgrad16_ws(const ConvGeom& g);
int mfma_wgrad16(const ConvGeom& g, const void* x, const void* dy, float* dw, float* db, void* ws,
                 size_t ws_bytes, hipStream_t s, int dtype);

}  // namespace flhip
