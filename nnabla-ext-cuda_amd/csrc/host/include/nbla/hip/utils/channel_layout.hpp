// ChannelLayout: how Group/InstanceNormalizationHip read a tensor with given
// batch axes and channel axis.  Channel-first (batch axes leading, channel axis
// right after them) and channel-last (batch axes leading, channel axis last)
// are read in place; every other layout goes to channel-first and back through
// an AxisAdaptor, as the reference does through the core's ChannelFirstAdaptor
// (group_normalization.cu:40-55, instance_normalization.cu:40-51).
#pragma once

#include <nbla/hip/utils/axis_adaptor.hpp>

namespace nbla {

struct ChannelLayout {
  bool channel_last = false;
  AxisAdaptor data;  // x, y, dy, dx
  // Tensors with one element per (batch index, channel or group) - statistics,
  // their gradients, per-sample parameters - are laid out by the caller in
  // axis order; the kernels want the batch axes first.  They differ only when
  // the channel axis precedes a batch axis.
  AxisAdaptor stats;
  Size_t batch = 1, channels = 1, spatial = 1;

  // stat_channels: extent of the channel position in the statistics (the
  // number of groups for GroupNormalization, of channels for
  // InstanceNormalization).
  void setup(const Shape_t &shape, const vector<int> &batch_axis, int c, Size_t stat_channels) {
    const int nb = static_cast<int>(batch_axis.size());
    const int ndim = static_cast<int>(shape.size());
    vector<int> b_sorted(batch_axis);
    std::sort(b_sorted.begin(), b_sorted.end());
    bool batch_leading = true;
    for (int b : b_sorted) batch_leading = batch_leading && b < nb;
    const bool channel_first = batch_leading && c == nb;
    channel_last = batch_leading && !channel_first && c == ndim - 1;
    channels = shape[c];
    batch = 1;
    Size_t total = 1;
    for (int b : b_sorted) batch *= shape[b];
    for (Size_t s : shape) total *= s;
    spatial = (batch > 0 && channels > 0) ? total / (batch * channels) : 0;
    vector<int> front(b_sorted);
    front.push_back(c);
    data.setup((channel_first || channel_last) ? Shape_t{total} : shape,
               (channel_first || channel_last) ? vector<int>{0} : front);
    // statistics: axes batch + channel in ascending order -> batch..., channel
    vector<int> kept(front);
    std::sort(kept.begin(), kept.end());
    Shape_t stat_shape;
    vector<int> stat_front;
    for (int b : b_sorted)
      stat_front.push_back(static_cast<int>(std::find(kept.begin(), kept.end(), b) - kept.begin()));
    stat_front.push_back(static_cast<int>(std::find(kept.begin(), kept.end(), c) - kept.begin()));
    for (int k : kept) stat_shape.push_back(k == c ? stat_channels : shape[k]);
    stats.setup(stat_shape, stat_front);
  }
};

} // namespace nbla
