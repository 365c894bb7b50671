/*
 * Test-only entry points of libmxq_hip.so.  They are exported by the library but are not
 * part of the operator contract (include/mxq.h): a test uses them to run one chosen kernel
 * variant on a shape of its choice.  Nothing is kept between calls; the choice is an
 * argument, never process state.
 */
#ifndef MXQ_TEST_HOOKS_H_
#define MXQ_TEST_HOOKS_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* mxq_quantized_fc with the launcher's choices pinned:
 *   cfg            tile configuration number (mxq_fc.hip lists them); 0 = choose by shape
 *   splits         work-groups per output tile along K; 0 = choose, 1 = none
 *   stream_groups  work-groups per CU of the short-K streaming kernel; 0 = choose
 * A pinned choice the shape does not qualify for is an error, not a fallback. */
int mxq_test_quantized_fc(void* stream, const int8_t* data, const int8_t* weight,
                          const int8_t* bias, int M, int N, int K, const float* min_data,
                          const float* max_data, const float* min_weight,
                          const float* max_weight, const float* min_bias, const float* max_bias,
                          int32_t* out32, float* omin, float* omax, int8_t* out8, float* rmin,
                          float* rmax, int relu, float min_calib, float max_calib,
                          void* workspace, size_t workspace_bytes, int cfg, int splits,
                          int stream_groups);

/* mxq_quantized_fc_f32 with the tile configuration and the split-K factor pinned. */
int mxq_test_quantized_fc_f32(void* stream, const int8_t* data, const int8_t* weight,
                              const int8_t* bias, int M, int N, int K, const float* min_data,
                              const float* max_data, const float* min_weight,
                              const float* max_weight, const float* min_bias,
                              const float* max_bias, float* out_f32, float* omin, float* omax,
                              float* rmin, float* rmax, int relu, float min_calib,
                              float max_calib, void* workspace, size_t workspace_bytes, int cfg,
                              int splits);

/* mxq_quantized_fc_sum with the tile configuration, the split-K factor and the streaming
 * kernel's work-groups per CU pinned. */
int mxq_test_quantized_fc_sum(void* stream, const int8_t* data, const int8_t* weight,
                              const int8_t* bias, int M, int N, int K, const float* min_data,
                              const float* max_data, const float* min_weight,
                              const float* max_weight, const float* min_bias,
                              const float* max_bias, const int8_t* residual,
                              const float* min_residual, const float* max_residual,
                              int8_t* out8, float* omin, float* omax, float* rmin, float* rmax,
                              float min_calib, float max_calib, float sum_min_calib,
                              float sum_max_calib, int sum_relu, void* workspace,
                              size_t workspace_bytes, int cfg, int splits, int stream_groups);

/* mxq_quantized_conv_nhwc with the tile configuration (mxq_conv.hip lists them) and the
 * split-K factor pinned. */
int mxq_test_quantized_conv_nhwc(void* stream, const int8_t* data, const int8_t* weight,
                                 const int8_t* bias, int N, int H, int W, int C, int O, int KH,
                                 int KW, int stride_h, int stride_w, int pad_h, int pad_w,
                                 int dilate_h, int dilate_w, const float* min_data,
                                 const float* max_data, const float* min_weight,
                                 const float* max_weight, const float* min_bias,
                                 const float* max_bias, int32_t* out32, float* omin,
                                 float* omax, int8_t* out8, float* rmin, float* rmax, int relu,
                                 float min_calib, float max_calib, void* workspace,
                                 size_t workspace_bytes, int cfg, int splits);

/* mxq_quantized_conv_nchw with its route pinned: cfg 1 = through the layout adapters,
 * 71 ... 84 = a tile of the NCHW 1x1 kernel (mxq_conv_nchw.hip lists them), 0 = choose. */
int mxq_test_quantized_conv_nchw(void* stream, const int8_t* data, const int8_t* weight,
                                 const int8_t* bias, int N, int C, int H, int W, int O, int KH,
                                 int KW, int stride_h, int stride_w, int pad_h, int pad_w,
                                 int dilate_h, int dilate_w, const float* min_data,
                                 const float* max_data, const float* min_weight,
                                 const float* max_weight, const float* min_bias,
                                 const float* max_bias, int32_t* out32, float* omin, float* omax,
                                 void* workspace, size_t workspace_bytes, int cfg);

#ifdef __cplusplus
}
#endif
#endif /* MXQ_TEST_HOOKS_H_ */
