// Minimal stand-in for the reference's graph runtime types, enough to compile
// and drive the MoE node classes outside the full engine.  Same names and
// member signatures as include/coalsack/core/graph_message.h and
// include/coalsack/image/frame_message.h of the reference (frame number and
// timestamp carried by result messages); no serialization, no registry.
#pragma once
#include <cstdint>
#include <memory>

#define COALSACK_REGISTER_NODE(...)
#define COALSACK_REGISTER_MESSAGE(...)

namespace coalsack {

class graph_message {
 public:
  virtual ~graph_message() = default;
};
using graph_message_ptr = std::shared_ptr<graph_message>;

class frame_message_base : public graph_message {
  uint64_t frame_number_ = 0;
  double timestamp_ = 0.0;

 public:
  uint64_t get_frame_number() const { return frame_number_; }
  void set_frame_number(uint64_t v) { frame_number_ = v; }
  double get_timestamp() const { return timestamp_; }
  void set_timestamp(double v) { timestamp_ = v; }
};

}  // namespace coalsack
