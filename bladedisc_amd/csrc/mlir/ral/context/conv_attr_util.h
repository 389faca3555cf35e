// TensorFlow-style convolution attributes -> the padding / metadata / result shape that
// ral_qconv takes.  Same rules as the reference's helpers
// (tao_compiler/mlir/ral/context/common_context_impl_quantization.h:27-206):
//   data_format  "NHWC" / "NCHW" (any permutation naming N and C); the other two
//                dimensions are the spatial ones, in order;
//   strides / dilations  1 value (both spatial dims), 2 values (spatial dims) or 4
//                values (indexed like the input's dimensions);
//   padding      "SAME" (TF rule: total = max(k_eff - (in % s ? in % s : s), 0), the
//                smaller half first), "VALID", or "EXPLICIT" with 4 values
//                (lo0, hi0, lo1, hi1) or 8 values (lo/hi per input dimension);
//   weights      [out_channels, filter_h, filter_w, in_channels] for every data_format;
//   result dim   (in + lo + hi - k*d + d + s - 1) / s.
#ifndef RAL_CONTEXT_CONV_ATTR_UTIL_H_
#define RAL_CONTEXT_CONV_ATTR_UTIL_H_

#include <cstdint>
#include <string>
#include <vector>

namespace tao {
namespace ral {

struct Conv2dPlan {
  int32_t padding[4];    // lo0, hi0, lo1, hi1
  int32_t metadata[17];  // input {N,C,S0,S1}, kernel {I,O,S0,S1}, output {N,C,S0,S1},
                         // strides[2], dilations[2], weight_is_const
  int64_t result_sizes[4];
};

// Returns an empty string on success, else what is wrong with the attributes.
inline std::string planConv2d(const std::string& data_format,
                              const std::vector<int64_t>& strides_attr,
                              const std::vector<int64_t>& dilations_attr,
                              const std::string& padding_attr,
                              const std::vector<int64_t>& explicit_paddings,
                              bool weight_is_const, const int64_t in_sizes[4],
                              const int64_t w_sizes[4], Conv2dPlan* plan) {
  if (data_format.size() != 4) return "data_format must name 4 dimensions";
  const size_t batch = data_format.find('N'), channel = data_format.find('C');
  if (batch == std::string::npos || channel == std::string::npos)
    return "data_format must contain N and C";
  int spatial[2], ns = 0;
  for (int i = 0; i < 4; ++i)
    if (i != (int)batch && i != (int)channel) {
      if (ns == 2) return "data_format must have two spatial dimensions";
      spatial[ns++] = i;
    }
  if (ns != 2) return "data_format must have two spatial dimensions";

  auto expand = [&](const std::vector<int64_t>& attr, int32_t out[2]) {
    if (attr.size() == 1) {
      out[0] = out[1] = (int32_t)attr[0];
    } else if (attr.size() == 2) {
      out[0] = (int32_t)attr[0];
      out[1] = (int32_t)attr[1];
    } else if (attr.size() == 4) {
      out[0] = (int32_t)attr[spatial[0]];
      out[1] = (int32_t)attr[spatial[1]];
    } else {
      return false;
    }
    return out[0] > 0 && out[1] > 0;
  };
  int32_t strides[2], dilations[2];
  if (!expand(strides_attr, strides)) return "strides must have 1, 2 or 4 positive entries";
  if (!expand(dilations_attr, dilations)) return "dilations must have 1, 2 or 4 positive entries";

  int32_t* pad = plan->padding;
  if (padding_attr == "VALID") {
    pad[0] = pad[1] = pad[2] = pad[3] = 0;
  } else if (padding_attr == "SAME") {
    for (int i = 0; i < 2; ++i) {
      const int64_t in = in_sizes[spatial[i]];
      const int64_t k_eff = (w_sizes[1 + i] - 1) * dilations[i] + 1;
      const int64_t rem = in % strides[i];
      int64_t total = k_eff - (rem == 0 ? strides[i] : rem);
      if (total < 0) total = 0;
      pad[2 * i] = (int32_t)(total / 2);
      pad[2 * i + 1] = (int32_t)(total - total / 2);
    }
  } else if (padding_attr == "EXPLICIT") {
    if (explicit_paddings.size() == 4) {
      for (int i = 0; i < 4; ++i) pad[i] = (int32_t)explicit_paddings[i];
    } else if (explicit_paddings.size() == 8) {
      for (int i = 0; i < 2; ++i) {
        pad[2 * i] = (int32_t)explicit_paddings[2 * spatial[i]];
        pad[2 * i + 1] = (int32_t)explicit_paddings[2 * spatial[i] + 1];
      }
    } else {
      return "explicit_paddings must have 4 or 8 entries";
    }
  } else {
    return "padding must be SAME, VALID or EXPLICIT";
  }

  int32_t* md = plan->metadata;
  const int32_t io_layout[4] = {(int32_t)batch, (int32_t)channel, spatial[0], spatial[1]};
  for (int i = 0; i < 4; ++i) md[i] = md[8 + i] = io_layout[i];
  md[4] = 3;  // kernel input features are the last dimension
  md[5] = 0;  // kernel output features the first
  md[6] = 1;
  md[7] = 2;
  md[12] = strides[0];
  md[13] = strides[1];
  md[14] = dilations[0];
  md[15] = dilations[1];
  md[16] = weight_is_const ? 1 : 0;

  for (int i = 0; i < 2; ++i) {
    const int64_t in = in_sizes[spatial[i]], k = w_sizes[1 + i];
    const int64_t s = strides[i], d = dilations[i];
    plan->result_sizes[spatial[i]] = (in + pad[2 * i] + pad[2 * i + 1] - k * d + d + s - 1) / s;
  }
  plan->result_sizes[batch] = in_sizes[batch];
  plan->result_sizes[channel] = w_sizes[0];
  return "";
}

}  // namespace ral
}  // namespace tao

#endif  // RAL_CONTEXT_CONV_ATTR_UTIL_H_
