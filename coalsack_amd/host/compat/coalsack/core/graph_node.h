// Stand-in for include/coalsack/core/graph_node.h:66-152: named inputs and
// outputs, and the process(input_name, message) entry an upstream edge calls.
#pragma once
#include <stdexcept>
#include <string>
#include <unordered_map>

#include "coalsack/core/graph_edge.h"

namespace coalsack {

class graph_node {
  std::unordered_map<std::string, graph_edge_ptr> outputs_, inputs_;

 public:
  virtual ~graph_node() = default;
  virtual std::string get_proc_name() const = 0;
  virtual void process(std::string input_name, graph_message_ptr message) {
    (void)input_name;
    (void)message;
  }
  void set_output(graph_edge_ptr output) { set_output(output, "default"); }
  void set_output(graph_edge_ptr output, std::string name) {
    output->set_name(name);
    outputs_[name] = output;
  }
  graph_edge_ptr get_output() const { return get_output("default"); }
  graph_edge_ptr get_output(std::string name) const {
    auto it = outputs_.find(name);
    if (it == outputs_.end()) throw std::invalid_argument("no such output: " + name);
    return it->second;
  }
  // Connecting an input subscribes this node's process() to the edge.
  void set_input(graph_edge_ptr input) { set_input(input, "default"); }
  void set_input(graph_edge_ptr input, std::string name) {
    inputs_[name] = input;
    input->subscribe([this, name](graph_message_ptr m) { this->process(name, m); });
  }
};

}  // namespace coalsack
