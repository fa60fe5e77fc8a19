// Stand-in for include/coalsack/nn/result_message.h:14-121: ok / error envelope
// around named message fields, carrying frame number and timestamp.
#pragma once
#include <memory>
#include <string>
#include <unordered_map>

#include "coalsack/core/graph_message.h"

namespace coalsack {

class result_message : public frame_message_base {
  bool ok_ = true;
  std::unordered_map<std::string, graph_message_ptr> fields_;
  std::string error_text_;

 public:
  using field_map = std::unordered_map<std::string, graph_message_ptr>;
  static std::shared_ptr<result_message> ok(const field_map& fields) {
    auto r = std::make_shared<result_message>();
    r->fields_ = fields;
    return r;
  }
  static std::shared_ptr<result_message> ok(const std::string& name, graph_message_ptr value) {
    return ok(field_map{{name, value}});
  }
  static std::shared_ptr<result_message> error(const field_map& fields, const std::string& message) {
    auto r = std::make_shared<result_message>();
    r->ok_ = false;
    r->fields_ = fields;
    r->error_text_ = message;
    return r;
  }
  void add_field(const std::string& name, graph_message_ptr m) { fields_[name] = m; }
  graph_message_ptr get_field(const std::string& name) const {
    auto it = fields_.find(name);
    return it == fields_.end() ? nullptr : it->second;
  }
  const field_map& get_fields() const { return fields_; }
  bool is_ok() const { return ok_; }
  bool is_error() const { return !ok_; }
  std::string get_error_message() const { return ok_ ? "" : error_text_; }
};

}  // namespace coalsack
