// Stand-in for include/coalsack/nn/nn_op_node.h:137-220 (binary_op_node) and :222-315
// (variadic_op_node): the bases that unpack named tensor fields from a
// result_message, call compute(), and send the result -- or the caught exception
// as an error result with a null field -- downstream.
#pragma once
#include <exception>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "coalsack/core/graph_edge.h"
#include "coalsack/core/graph_node.h"
#include "coalsack/nn/result_message.h"
#include "coalsack/tensor/dynamic_tensor.h"
#include "coalsack/tensor/dynamic_tensor_message.h"

namespace coalsack {

inline dynamic_tensor get_tensor_from_result_message(const std::shared_ptr<result_message>& msg,
                                                     const std::string& field_name) {
  auto t = std::dynamic_pointer_cast<dynamic_tensor_message>(msg->get_field(field_name));
  if (!t) throw std::runtime_error("Field '" + field_name + "' is not a dynamic_tensor_message");
  return t->get_tensor();
}

class binary_op_node : public graph_node {
 protected:
  graph_edge_ptr output_;
  std::string node_name_, op_type_, input_a_name_, input_b_name_, output_name_;
  virtual dynamic_tensor compute(const dynamic_tensor& a, const dynamic_tensor& b) = 0;

 public:
  explicit binary_op_node(const std::string& op_type)
      : output_(std::make_shared<graph_edge>(this)), op_type_(op_type) {
    set_output(output_);
  }
  std::string get_proc_name() const override { return "nn_" + op_type_; }
  void set_input_names(const std::string& a, const std::string& b) {
    input_a_name_ = a;
    input_b_name_ = b;
  }
  void set_output_name(const std::string& name) { output_name_ = name; }
  void set_node_name(const std::string& name) { node_name_ = name; }
  std::vector<std::string> get_input_names() const { return {input_a_name_, input_b_name_}; }

  void process(std::string /*input_name*/, graph_message_ptr message) override {
    auto in = std::dynamic_pointer_cast<result_message>(message);
    const uint64_t frame = in ? in->get_frame_number() : 0;
    std::shared_ptr<result_message> out;
    if (in && !in->is_ok()) {
      out = result_message::error({{output_name_, nullptr}}, "Input error");
    } else {
      try {
        dynamic_tensor a, b;
        if (in) {
          if (input_a_name_.empty() || input_b_name_.empty())
            throw std::runtime_error(op_type_ + ": input names not set");
          a = get_tensor_from_result_message(in, input_a_name_);
          b = get_tensor_from_result_message(in, input_b_name_);
        }
        out = result_message::ok({{output_name_, std::make_shared<dynamic_tensor_message>(compute(a, b))}});
      } catch (const std::exception& e) {
        out = result_message::error({{output_name_, nullptr}}, e.what());
      }
    }
    out->set_frame_number(frame);
    output_->send(out);
  }
};

class variadic_op_node : public graph_node {
 protected:
  graph_edge_ptr output_;
  std::string op_type_;
  std::vector<std::string> input_names_;
  std::string output_name_, node_name_;
  virtual dynamic_tensor compute(const std::vector<dynamic_tensor>& inputs) = 0;

 public:
  variadic_op_node(const std::string& op_type, size_t /*num_inputs*/)
      : output_(std::make_shared<graph_edge>(this)), op_type_(op_type) {
    set_output(output_);
  }
  std::string get_proc_name() const override { return "nn_" + op_type_; }
  void set_input_names(const std::vector<std::string>& names) { input_names_ = names; }
  void set_output_name(const std::string& name) { output_name_ = name; }
  void set_node_name(const std::string& name) { node_name_ = name; }
  std::vector<std::string> get_input_names() const { return input_names_; }
  std::string get_output_name() const { return output_name_; }

  void process(std::string /*input_name*/, graph_message_ptr message) override {
    auto in = std::dynamic_pointer_cast<result_message>(message);
    const uint64_t frame = in ? in->get_frame_number() : 0;
    std::shared_ptr<result_message> out;
    if (in && !in->is_ok()) {
      out = result_message::error({{output_name_, nullptr}}, "Input error");
    } else {
      try {
        std::vector<dynamic_tensor> inputs;
        if (in) {
          if (input_names_.empty()) throw std::runtime_error(op_type_ + ": input_names_ not set");
          for (const auto& name : input_names_) {
            if (name.empty()) throw std::runtime_error(op_type_ + ": input_name is empty");
            inputs.push_back(get_tensor_from_result_message(in, name));
          }
        }
        out = result_message::ok({{output_name_, std::make_shared<dynamic_tensor_message>(compute(inputs))}});
      } catch (const std::exception& e) {
        out = result_message::error({{output_name_, nullptr}}, e.what());
      }
    }
    out->set_frame_number(frame);
    output_->send(out);
  }
};

}  // namespace coalsack
