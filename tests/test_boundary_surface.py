"""The drop-in node headers are compiled here against small stand-ins of the reference's
interface headers.  This test holds the stand-ins -- and through them the nodes -- to the
reference: every declaration the nodes rely on must appear, with the same signature, both in
the reference header and in the stand-in of the same relative path; and every member the
node headers call on those types must be one of the declarations so checked.  The first
part needs the reference tree and is skipped where it is absent."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference/include/coalsack"
COMPAT = os.path.join(ROOT, "coalsack_amd", "host", "compat", "coalsack")
NODES = os.path.join(ROOT, "coalsack_amd", "host", "nodes", "coalsack", "nn", "nn_ops")

# header (relative to include/coalsack) -> {member name: signature as a whitespace-free regex}
SURFACE = {
    "nn/nn_op_node.h": {
        "get_tensor_from_result_message":
            r"inlinedynamic_tensorget_tensor_from_result_message\(conststd::shared_ptr<result_message>&\w+,conststd::string&\w+\)",
        "binary_op_node": r"classbinary_op_node:publicgraph_node\{",
        "binary_op_node()": r"explicitbinary_op_node\(conststd::string&op_type\)",
        "binary compute": r"virtualdynamic_tensorcompute\(constdynamic_tensor&a,constdynamic_tensor&b\)=0;",
        "variadic_op_node": r"classvariadic_op_node:publicgraph_node\{",
        "variadic_op_node()": r"variadic_op_node\(conststd::string&op_type,size_t(/\*)?num_inputs(\*/)?\)",
        "variadic compute": r"virtualdynamic_tensorcompute\(conststd::vector<dynamic_tensor>&inputs\)=0;",
        "set_input_names": r"voidset_input_names\(conststd::vector<std::string>&names\)",
        "set_input_names(a,b)": r"voidset_input_names\(conststd::string&a,conststd::string&b\)",
        "set_output_name": r"voidset_output_name\(conststd::string&name\)",
        "set_node_name": r"voidset_node_name\(conststd::string&name\)",
        "get_input_names": r"std::vector<std::string>get_input_names\(\)const",
        "get_output_name": r"std::stringget_output_name\(\)const",
        "get_proc_name": r"std::stringget_proc_name\(\)constoverride\{return\"nn_\"\+op_type_;\}",
        "output_": r"graph_edge_ptroutput_;",
        "input_names_": r"std::vector<std::string>input_names_;",
        "output_name_": r"std::string(\w+,)*output_name_[;,]",
        "process": r"voidprocess\((\[\[maybe_unused\]\])?std::string(/\*)?input_name(\*/)?,graph_message_ptrmessage\)override",
    },
    "nn/result_message.h": {
        "ok": r"staticstd::shared_ptr<result_message>ok\(conststd::unordered_map<std::string,graph_message_ptr>&fields\)|"
              r"usingfield_map=std::unordered_map<std::string,graph_message_ptr>;staticstd::shared_ptr<result_message>ok\(constfield_map&fields\)",
        "error": r"staticstd::shared_ptr<result_message>error\(const(std::unordered_map<std::string,graph_message_ptr>|field_map)&fields,conststd::string&\w+\)",
        "get_field": r"graph_message_ptrget_field\(conststd::string&name\)const",
        "get_fields": r"const(std::unordered_map<std::string,graph_message_ptr>|field_map)&get_fields\(\)const",
        "is_ok": r"boolis_ok\(\)const",
        "is_error": r"boolis_error\(\)const",
        "get_error_message": r"std::stringget_error_message\(\)const",
        "base": r"classresult_message:publicframe_message_base\{",
    },
    "tensor/dynamic_tensor.h": {
        "dtype": r"enumclassdtype\{float32,float16,int64,int32,bool_,uint8,float64,?\};",
        "ctor": r"dynamic_tensor\(dtypedt,conststd::vector<int64_t>&shape\)",
        "ctor data": r"dynamic_tensor\(dtypedt,conststd::vector<int64_t>&shape,constvoid\*data\)",
        "get_dtype": r"dtypeget_dtype\(\)const",
        "shape": r"conststd::vector<int64_t>&shape\(\)const",
        "ndim": r"int64_tndim\(\)const",
        "dim": r"int64_tdim\(int64_ti\)const",
        "numel": r"int64_tnumel\(\)const",
        "bytes": r"size_tbytes\(\)const",
        "data_ptr": r"template<(typename|class)T>constT\*data_ptr\(\)const",
        "data_ptr mutable": r"template<(typename|class)T>T\*data_ptr\(\)\{",
        "broadcast_shape": r"staticstd::vector<int64_t>broadcast_shape\(conststd::vector<int64_t>&\w+,conststd::vector<int64_t>&\w+\)",
        "empty": r"boolempty\(\)const",
    },
    "tensor/dynamic_mx_tensor.h": {
        "ctor": r"explicitdynamic_mx_tensor\(conststd::vector<int64_t>&shape\)",
        "ndim": r"size_tndim\(\)const",
        "dim": r"int64_tdim\(size_t\w+\)const",
        "shape": r"conststd::vector<int64_t>&shape\(\)const",
        "size_bytes": r"size_tsize_bytes\(\)const",
        "num_blocks": r"size_tnum_blocks\(\)const",
        "data_ptr": r"constuint8_t\*data_ptr\(\)const",
        "data_ptr mutable": r"uint8_t\*data_ptr\(\)\{",
    },
    "tensor/dynamic_tensor_message.h": {
        "ctor": r"explicitdynamic_tensor_message\(constdynamic_tensor&\w+\)",
        "get_tensor": r"constdynamic_tensor&get_tensor\(\)const",
        "base": r"classdynamic_tensor_message:publicgraph_message\{",
    },
    "tensor/dynamic_mx_tensor_message.h": {
        "ctor": r"explicitdynamic_mx_tensor_message\(constdynamic_mx_tensor&\w+\)",
        "get_mx_tensor": r"constdynamic_mx_tensor&get_mx_tensor\(\)const",
        "base": r"classdynamic_mx_tensor_message:publicgraph_message\{",
    },
    "core/graph_node.h": {
        "get_proc_name": r"virtualstd::stringget_proc_name\(\)const=0;",
        "process": r"virtualvoidprocess\((\[\[maybe_unused\]\])?std::stringinput_name,(\[\[maybe_unused\]\])?graph_message_ptrmessage\)",
        "set_output": r"voidset_output\(graph_edge_ptroutput\)",
        "get_output": r"graph_edge_ptrget_output\(\)const",
        "set_input": r"voidset_input\(graph_edge_ptrinput\)",
    },
    "core/graph_edge.h": {
        "send": r"voidsend\(graph_message_ptrmessage\)",
        "ctor": r"graph_edge\(graph_node\*source",
        "ptr": r"usinggraph_edge_ptr=std::shared_ptr<graph_edge>;",
    },
}
# frame number / timestamp accessors live in another header of the reference
FRAME_REF = ("image/frame_message.h", "core/graph_message.h", {
    "get_frame_number": r"uint64_tget_frame_number\(\)const",
    "set_frame_number": r"voidset_frame_number\(uint64_t\w+\)",
    "get_timestamp": r"\w+get_timestamp\(\)const",
    "set_timestamp": r"voidset_timestamp\(\w+\w+\)",
})


def squeeze(path):
    text = open(path).read()
    text = re.sub(r"//[^\n]*", "", text)
    text = re.sub(r"/\*(?!num_inputs\*/|input_name\*/).*?\*/", "", text, flags=re.S)
    return re.sub(r"\s+", "", text)


def check(header_text, table, where):
    missing = [name for name, rx in table.items() if not re.search(rx, header_text)]
    assert not missing, f"{where}: no declaration matching {missing}"


@pytest.mark.parametrize("rel", sorted(SURFACE))
def test_stand_in_declares_the_surface(rel):
    check(squeeze(os.path.join(COMPAT, rel)), SURFACE[rel], "stand-in " + rel)


@pytest.mark.skipif(not os.path.isdir(REF), reason="reference tree not present")
@pytest.mark.parametrize("rel", sorted(SURFACE))
def test_reference_declares_the_same_surface(rel):
    check(squeeze(os.path.join(REF, rel)), SURFACE[rel], "reference " + rel)


def test_frame_accessors():
    ref_rel, compat_rel, table = FRAME_REF
    check(squeeze(os.path.join(COMPAT, compat_rel)), table, "stand-in " + compat_rel)
    if os.path.isdir(REF):
        check(squeeze(os.path.join(REF, ref_rel)), table, "reference " + ref_rel)


# what the node headers may call with . or -> : the checked surface, the C++ library, and
# the nodes' own helpers
CHECKED = {"get_dtype", "shape", "ndim", "dim", "numel", "bytes", "data_ptr", "empty", "size_bytes", "num_blocks",
           "get_field", "get_fields", "is_ok", "is_error", "get_error_message", "get_frame_number",
           "set_frame_number", "get_timestamp", "set_timestamp", "send", "get_tensor", "get_mx_tensor"}
LIBRARY = {"size", "push_back", "emplace_back", "begin", "end", "empty", "data", "what", "resize", "find", "count",
           "c_str", "back", "reserve", "assign", "clear", "lock", "reset", "expired", "erase"}
# the nodes' own helpers: resident_weight.h's slots, moe_block_context.h's frame bookkeeping
OWN = {"get", "split", "frame_matches", "publish", "unpublish", "usable"}


def test_nodes_call_nothing_outside_the_checked_surface():
    for name in sorted(os.listdir(NODES)):
        text = open(os.path.join(NODES, name)).read()
        text = re.sub(r"//[^\n]*", "", text)
        text = re.sub(r'"(\\.|[^"\\])*"', '""', text)
        called = set(re.findall(r"(?:\.|->)\s*(?:template\s+)?(\w+)\s*(?:<[^<>()]*>)?\s*\(", text))
        stray = called - CHECKED - LIBRARY - OWN
        assert not stray, f"{name} calls {sorted(stray)}: add the declaration to SURFACE or drop the call"


def test_node_classes_keep_the_reference_names_and_registration():
    expect = {"moe_router_node.h": ("moe_router_node", "variadic_op_node"),
              "expert_mlp_node.h": ("expert_mlp_node", "graph_node"),
              "expert_merge_node.h": ("expert_merge_node", "variadic_op_node"),
              "dense_ffn_node.h": ("dense_ffn_node", "variadic_op_node"),
              "matmul_transpose_mixed_node.h": ("matmul_transpose_mixed_node", "binary_op_node"),
              "rmsnorm_node.h": ("rmsnorm_node", "binary_op_node"),
              "add_node.h": ("add_node", "binary_op_node")}
    for name, (cls, base) in expect.items():
        ours = squeeze(os.path.join(NODES, name))
        decl = rf"class{cls}:public{base}\{{"
        reg = rf"COALSACK_REGISTER_NODE\(coalsack::{cls},coalsack::graph_node\)"
        assert re.search(decl, ours) and re.search(reg, ours), name
        if os.path.isdir(REF):
            theirs = squeeze(os.path.join(REF, "nn", "nn_ops", name))
            assert re.search(decl, theirs) and re.search(reg, theirs), "reference " + name
