// Host-side self test of the C ABI's argument handling, for a build of the host code with
// AddressSanitizer and UndefinedBehaviorSanitizer (`make sanitize`): every call here is answered on
// the host -- rejected before any launch, or a pure size query -- so it runs without a GPU.
// It walks the validation of every entry point (null pointers, bad shapes, bad dtype tags, sizes at
// and beyond the 32-bit limits, short workspaces) and the workspace / launch-shape arithmetic over a
// sweep of geometries, where an overflowing int or an out-of-range table index would show.
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <initializer_list>

#include "../../include/dk_hip.h"

static int failures = 0;
#define EXPECT(cond)                                                        \
  do {                                                                      \
    if (!(cond)) { std::printf("line %d: %s\n", __LINE__, #cond); ++failures; } \
  } while (0)

static dk_conv_desc conv(int n, int c, int h, int w, int k, int s, int p, int d, int scope, int groups, int dtype) {
  dk_conv_desc v;
  std::memset(&v, 0, sizeof v);
  v.batch = n, v.channel = c, v.in_h = h, v.in_w = w;
  v.k_h = v.k_w = k, v.stride_h = v.stride_w = s, v.pad_h = v.pad_w = p, v.dil_h = v.dil_w = d;
  v.scope_h = v.scope_w = scope, v.groups = groups, v.dtype = dtype;
  return v;
}

int main() {
  void* one = reinterpret_cast<void*>(16);  // never dereferenced: every call below is refused first
  const dk_conv_desc ok = conv(1, 4, 8, 8, 3, 1, 1, 1, 4, 1, DK_F32);
  int32_t oh = 0, ow = 0;
  EXPECT(dk_conv_out_size(&ok, &oh, &ow) == DK_OK && oh == 8 && ow == 8);
  EXPECT(dk_conv_out_size(nullptr, &oh, &ow) == DK_ERR_NULL_POINTER);

  // null tensors, every entry point
  EXPECT(dk_sample_depthwise_forward(&ok, nullptr, one, one, one, nullptr) == DK_ERR_NULL_POINTER);
  EXPECT(dk_sample_depthwise_backward_data(&ok, one, nullptr, one, one, nullptr) == DK_ERR_NULL_POINTER);
  EXPECT(dk_sample_depthwise_backward_filter(&ok, one, one, one, nullptr, one, 1 << 20, nullptr) == DK_ERR_NULL_POINTER);
  EXPECT(dk_sample_depthwise_backward_filter_static(&ok, one, one, nullptr, one, nullptr) == DK_ERR_NULL_POINTER);
  EXPECT(dk_sample_depthwise_backward_rotation(&ok, one, one, one, one, nullptr, one, 1 << 20, nullptr) == DK_ERR_NULL_POINTER);
  EXPECT(dk_sample_depthwise_backward(&ok, nullptr, one, one, one, one, one, one, one, 1 << 20, nullptr) == DK_ERR_NULL_POINTER);
  EXPECT(dk_deformable_sample_depthwise_forward(&ok, one, nullptr, one, one, one, nullptr) == DK_ERR_NULL_POINTER);
  EXPECT(dk_deformable_sample_depthwise_backward_data(&ok, one, one, one, one, nullptr, one, 1 << 20, nullptr) == DK_ERR_NULL_POINTER);
  EXPECT(dk_deformable_sample_depthwise_backward_filter(&ok, one, one, one, one, nullptr, one, 1 << 20, nullptr) == DK_ERR_NULL_POINTER);
  EXPECT(dk_deformable_sample_depthwise_backward_offset(&ok, one, one, one, one, one, nullptr, one, 1 << 20, nullptr) == DK_ERR_NULL_POINTER);
  EXPECT(dk_deformable_sample_depthwise_backward_rotation(&ok, one, one, one, one, one, nullptr, one, 1 << 20, nullptr) == DK_ERR_NULL_POINTER);
  EXPECT(dk_deformable_sample_depthwise_backward_offset_rotation(&ok, one, one, one, nullptr, one, one, one, one, 1 << 20, nullptr) == DK_ERR_NULL_POINTER);
  EXPECT(dk_deformable_sample_depthwise_backward_offset_rotation(&ok, one, one, one, one, one, one, nullptr, one, 1 << 20, nullptr) == DK_ERR_NULL_POINTER);

  // shapes
  dk_conv_desc bad = ok;
  bad.groups = 3;
  EXPECT(dk_conv_out_size(&bad, nullptr, nullptr) == DK_ERR_BAD_SHAPE);
  bad = conv(1, 4, 2, 2, 5, 1, 0, 1, 4, 1, DK_F32);
  EXPECT(dk_conv_out_size(&bad, nullptr, nullptr) == DK_ERR_BAD_SHAPE);
  bad = ok, bad.dtype = 9;
  EXPECT(dk_conv_out_size(&bad, nullptr, nullptr) == DK_ERR_BAD_DTYPE);
  bad = ok, bad.rotation_clip = 3;
  EXPECT(dk_conv_out_size(&bad, nullptr, nullptr) == DK_ERR_BAD_SHAPE);
  bad = ok, bad.rotation_clip = DK_CLIP_ROTATION, bad.clip_min = 1.f, bad.clip_max = 0.f;
  EXPECT(dk_conv_out_size(&bad, nullptr, nullptr) == DK_ERR_BAD_SHAPE);
  bad = ok, bad.stride_w = 0;
  EXPECT(dk_conv_out_size(&bad, nullptr, nullptr) == DK_ERR_BAD_SHAPE);
  bad = conv(4096, 4096, 512, 512, 3, 1, 1, 1, 4, 1, DK_F32);
  EXPECT(dk_conv_out_size(&bad, nullptr, nullptr) == DK_ERR_TOO_LARGE);
  bad = conv(INT32_MAX, INT32_MAX, INT32_MAX, INT32_MAX, INT32_MAX, INT32_MAX, INT32_MAX, INT32_MAX, INT32_MAX, 1, DK_F32);
  EXPECT(dk_conv_out_size(&bad, nullptr, nullptr) < 0);
  bad = conv(1, 1, INT32_MAX, 1, 3, 1, INT32_MAX, 1, 4, 1, DK_F32);  // in + 2 * pad overflows 32 bits
  EXPECT(dk_conv_out_size(&bad, nullptr, nullptr) < 0);

  // a workspace one byte short
  const size_t need = dk_sample_depthwise_backward_filter_workspace(&ok);
  EXPECT(need > 0);
  EXPECT(dk_sample_depthwise_backward_filter(&ok, one, one, one, one, one, need - 1, nullptr) == DK_ERR_WORKSPACE);
  EXPECT(dk_sample_depthwise_backward_filter(&ok, one, one, one, one, nullptr, need, nullptr) == DK_ERR_WORKSPACE);

  // the static-scratch entry point refuses what exceeds its buffer
  const dk_conv_desc big = conv(8, 1024, 14, 14, 3, 1, 1, 1, 5, 1, DK_F32);
  EXPECT(dk_sample_depthwise_backward_filter_workspace(&big) > DK_STATIC_SCRATCH_BYTES);
  EXPECT(dk_sample_depthwise_backward_filter_static(&big, one, one, one, one, nullptr) == DK_ERR_SCRATCH_LIMIT);

  // size queries over a sweep of geometries: launch-shape arithmetic only
  size_t total = 0;
  for (int dtype = DK_F32; dtype <= DK_F64; ++dtype)
    for (int scope = 2; scope <= 9; ++scope)
      for (int stride = 1; stride <= 2; ++stride)
        for (int hw : {1, 3, 7, 14, 28, 56, 57, 112, 130, 224, 1000})
          for (int c : {1, 3, 16, 36, 144, 960, 4096})
            for (int n : {0, 1, 7, 64}) {
              const int groups = c % 3 == 0 ? 3 : 1;
              const dk_conv_desc d = conv(n, c, hw, hw + hw % 3, 3, stride, 1, 1, scope, groups, dtype);
              if (dk_conv_out_size(&d, &oh, &ow) != DK_OK) continue;
              total += dk_sample_depthwise_backward_filter_workspace(&d) + dk_sample_depthwise_backward_rotation_workspace(&d) +
                       dk_sample_depthwise_backward_workspace(&d) + dk_deformable_sample_depthwise_backward_data_workspace(&d) +
                       dk_deformable_sample_depthwise_backward_filter_workspace(&d) +
                       dk_deformable_sample_depthwise_backward_offset_workspace(&d) +
                       dk_deformable_sample_depthwise_backward_rotation_workspace(&d) +
                       dk_deformable_sample_depthwise_backward_offset_rotation_workspace(&d);
            }
  EXPECT(total > 0);

  // N-d sampler
  dk_nd_desc nd;
  std::memset(&nd, 0, sizeof nd);
  nd.batch = 4, nd.channel = 2, nd.dims = 9, nd.dtype = DK_F32;
  EXPECT(dk_nd_linear_sample_forward(&nd, one, one, nullptr, one, nullptr, 0, nullptr) == DK_ERR_UNSUPPORTED);
  nd.dims = 3, nd.shape[0] = nd.shape[1] = 4, nd.shape[2] = 0;
  EXPECT(dk_nd_linear_sample_forward(&nd, one, one, nullptr, one, nullptr, 0, nullptr) == DK_ERR_BAD_SHAPE);
  nd.shape[0] = nd.shape[1] = nd.shape[2] = 2000;
  EXPECT(dk_nd_linear_sample_forward(&nd, one, one, nullptr, one, nullptr, 0, nullptr) == DK_ERR_TOO_LARGE);
  nd.shape[0] = nd.shape[1] = nd.shape[2] = 32, nd.channel = 64;
  for (int64_t b : {int64_t(0), int64_t(1), int64_t(4096), int64_t(1) << 20, int64_t(1) << 34}) {
    nd.batch = b;
    total += dk_nd_linear_sample_forward_workspace(&nd) + dk_nd_linear_sample_order_bytes(&nd) +
             dk_nd_linear_sample_order_workspace(&nd) + dk_nd_linear_sample_backward_data_workspace(&nd) +
             dk_nd_linear_sample_backward_coord_workspace(&nd);
  }
  nd.batch = 4;
  EXPECT(dk_nd_linear_sample_forward(&nd, nullptr, one, nullptr, one, nullptr, 0, nullptr) == DK_ERR_NULL_POINTER);

  // offset branch
  dk_offset_conv_desc oc = {64, 144, 18, 56, 56, DK_F32};
  EXPECT(dk_offset_conv_supported(&oc) == 1);
  EXPECT(dk_offset_conv_forward(&oc, nullptr, one, one, one, one, 1 << 30, nullptr) == DK_ERR_NULL_POINTER);
  EXPECT(dk_offset_conv_forward(&oc, one, one, one, one, one, 0, nullptr) == DK_ERR_WORKSPACE);
  oc.w = 57;
  EXPECT(dk_offset_conv_supported(&oc) == 0);
  EXPECT(dk_offset_conv_forward(&oc, one, one, one, one, one, 1 << 30, nullptr) == DK_ERR_UNSUPPORTED);
  EXPECT(dk_offset_conv_backward_bias(nullptr, one, one, one, 0, nullptr) == DK_ERR_NULL_POINTER);
  // the input gradient: planes 7 .. 112 wide; float32 tensors as bfloat16 pairs unless that is switched off
  oc.w = 56;
  EXPECT(dk_offset_conv_backward_input_workspace(&oc) > 0);
  EXPECT(dk_offset_conv_backward_input_worthwhile(&oc) == 1);
  EXPECT(dk_offset_conv_backward_input(&oc, one, one, one, one, 0, nullptr) == DK_ERR_WORKSPACE);
  oc.in_channels = 32;
  EXPECT(dk_offset_conv_backward_input_workspace(&oc) > 0);
  EXPECT(dk_offset_conv_backward_input_worthwhile(&oc) == 0);  // covered, but not the faster choice
  oc.in_channels = 144;
  {
    const unsigned pairs_off = 1u << 18;  // DK_NO_OFFSET_PAIRS
    const unsigned before = dk_test_switches(pairs_off);
    EXPECT(dk_offset_conv_supported(&oc) == 1);  // the fp32 matrix-instruction forward
    EXPECT(dk_offset_conv_backward_input_workspace(&oc) == 0);
    EXPECT(dk_offset_conv_backward_input(&oc, one, one, one, one, 1 << 30, nullptr) == DK_ERR_UNSUPPORTED);
    dk_test_switches(before);
  }
  oc.dtype = DK_BF16;
  EXPECT(dk_offset_conv_backward_input_workspace(&oc) > 0);
  EXPECT(dk_offset_conv_forward_workspace(&oc) > 0);
  EXPECT(dk_offset_conv_backward_input(&oc, nullptr, one, one, one, 1 << 30, nullptr) == DK_ERR_NULL_POINTER);
  EXPECT(dk_offset_conv_backward_input(&oc, one, one, one, one, 0, nullptr) == DK_ERR_WORKSPACE);
  oc.w = oc.h = 14;
  EXPECT(dk_offset_conv_backward_input_workspace(&oc) > 0);
  oc.w = 21;
  EXPECT(dk_offset_conv_backward_input(&oc, one, one, one, one, 1 << 30, nullptr) == DK_ERR_UNSUPPORTED);
  oc.w = 14;
  // stride 2: every pass on the 16-bit matrix instructions
  oc.w = oc.h = 56, oc.stride = 2;
  EXPECT(dk_offset_conv_supported(&oc) == 1);
  EXPECT(dk_offset_conv_forward_workspace(&oc) > 0);
  EXPECT(dk_offset_conv_forward(&oc, one, one, one, one, one, 0, nullptr) == DK_ERR_WORKSPACE);
  EXPECT(dk_offset_conv_backward_input_workspace(&oc) > 0);
  EXPECT(dk_offset_conv_backward_input(&oc, one, one, one, one, 0, nullptr) == DK_ERR_WORKSPACE);
  EXPECT(dk_offset_conv_backward_weight_workspace(&oc) > 0);
  EXPECT(dk_offset_conv_backward_weight(&oc, one, one, one, one, 0, nullptr) == DK_ERR_WORKSPACE);
  {
    const unsigned before = dk_test_switches(1u << 19);  // DK_NO_OFFSET_WGRAD16
    EXPECT(dk_offset_conv_backward_weight_workspace(&oc) == 0);
    EXPECT(dk_offset_conv_backward_weight(&oc, one, one, one, one, 1 << 30, nullptr) == DK_ERR_UNSUPPORTED);
    dk_test_switches(before);
  }
  oc.dtype = DK_F32;
  EXPECT(dk_offset_conv_supported(&oc) == 1);
  EXPECT(dk_offset_conv_backward_input_workspace(&oc) > 0);
  EXPECT(dk_offset_conv_backward_weight_workspace(&oc) > 0);
  oc.dtype = DK_BF16, oc.stride = 3;
  EXPECT(dk_offset_conv_forward(&oc, one, one, one, one, one, 1 << 30, nullptr) == DK_ERR_BAD_SHAPE);
  oc.stride = 0, oc.w = oc.h = 14;
  // the weight gradient: up to 20 outputs on the 16-bit matrix instructions, 15 and more on the fp32 ones
  EXPECT(dk_offset_conv_backward_weight_workspace(&oc) > 0);
  oc.out_channels = 7;
  EXPECT(dk_offset_conv_supported(&oc) == 1);
  EXPECT(dk_offset_conv_backward_weight_workspace(&oc) > 0);
  {
    const unsigned before = dk_test_switches(1u << 19);
    EXPECT(dk_offset_conv_backward_weight_workspace(&oc) == 0);
    EXPECT(dk_offset_conv_backward_weight(&oc, one, one, one, one, 1 << 30, nullptr) == DK_ERR_UNSUPPORTED);
    dk_test_switches(before);
  }

  EXPECT(std::strstr(dk_status_string(DK_ERR_WORKSPACE), "workspace") != nullptr);
  EXPECT(dk_status_string(-99) != nullptr);
  EXPECT(dk_test_switches(dk_test_switches(0)) == 0);  // set to 0, then restore: the second call returns the 0
  if (failures == 0) std::printf("abi selftest ok\n");
  return failures != 0;
}
