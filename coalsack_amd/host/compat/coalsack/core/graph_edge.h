// Stand-in for include/coalsack/core/graph_edge.h: an edge fans a message out,
// synchronously and in subscription order, to the callbacks registered on it
// (graph_edge.h:87-93 of the reference).
#pragma once
#include <functional>
#include <memory>
#include <string>
#include <vector>

#include "coalsack/core/graph_message.h"

namespace coalsack {

class graph_node;

class graph_edge {
  graph_node* source_;
  std::string name_;
  std::vector<std::function<void(graph_message_ptr)>> subscribers_;

 public:
  explicit graph_edge(graph_node* source) : source_(source) {}
  void set_name(std::string name) { name_ = std::move(name); }
  std::string get_name() const { return name_; }
  graph_node* get_source() const { return source_; }
  void subscribe(std::function<void(graph_message_ptr)> fn) { subscribers_.push_back(std::move(fn)); }
  void send(graph_message_ptr message) {
    for (auto& fn : subscribers_) fn(message);
  }
};
using graph_edge_ptr = std::shared_ptr<graph_edge>;

}  // namespace coalsack
