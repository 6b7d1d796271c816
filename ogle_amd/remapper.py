"""Graph pass over a .dlx model: folds BatchNormalization, and a following Relu / Clip,
into the convolution in front of them.

Restates converter/converter/optimizers/remapper.cc:36-176 of the reference on the
serialized ModelProto:

  Conv -> BatchNormalization                 =>  Conv (scaled filter, new bias)
  Conv -> BatchNormalization -> Relu | Clip  =>  Conv with activation_type / max set

  scale = gamma / sqrt(var + eps)         (fp32, remapper.cc:142-149)
  W[o]  *= scale[o]
  b[o]   = b[o] * scale[o] + (beta[o] - scale[o] * mean[o])   (a zero bias is made first
                                                                if the conv had none)
  Relu: activation_type "Relu", min = max = 0;  Clip: activation_type "Clip",
  max = clip.max and min left at 0 (remapper.cc:153-176), i.e. ReLU6 is Clip with max 6.

The fused node takes the name and the output tensor of the last node of the pattern, so
consumers are untouched.  Unlike the reference, a pattern is only folded when the
intermediate tensors have no other consumer and the parameters are constants owned by
the pattern; anything else is left as it is.

Node order and tensor indices of the result follow the reference's round trip through
its Graph class (converter/converter/core/converter.cc:33-42):

  1. GraphConstructor::Convert (graph/graph_constructor.cc:144-190) gives node ids in
     topological order, always taking the ready node that comes first in the file, so a
     file that is already sorted keeps its order and an unsorted one is sorted;
  2. the pass walks the ids from the last to the first; a bias it has to make is a new
     Const node named "<conv>:<input slot>" whose id is the next free one
     (remapper.cc:71-96), i.e. after every node of the file;
  3. Graph::ToGraphDef (graph/graph.cc:12-54, 233-331) sorts again, always taking the
     ready node with the smallest id, drops every node that has neither inputs nor
     consumers and is not a graph output (the folded BatchNormalization's parameters),
     and numbers the tensors in the order their nodes are written.

A made bias therefore comes after all other constants, and its convolution (with
everything downstream) after it.  One difference is kept on purpose: ToGraphDef only
lists a node as a graph output when it has no output slot (graph.cc:279-285), which is
never the case for a converted model, so the reference writes an empty output list;
here the output names of the source model are kept.
"""
import struct
from collections import defaultdict

import numpy as np

from . import dlx


def _decode_floats(buf, fields):
    out = {name: 0.0 for name in fields.values()}
    for field, wt, v in dlx._fields(buf):
        if field in fields and wt == 5:
            out[fields[field]] = struct.unpack("<f", v)[0]
    return out


def _const_tensor(node):
    for field, wt, v in dlx._fields(node["attr"][dlx.ATTR_CONST]):
        if field == 1:
            return dlx.decode_tensor(v)
    raise ValueError("Const node %r has no value" % node["name"])


def _set_const(node, tensor, values):
    node["attr"][dlx.ATTR_CONST] = dlx._sub(1, dlx.encode_tensor(
        np.asarray(values, np.float32).reshape(-1), tensor["dims"], tensor["data_format"],
        tensor["target_data_format"]))


def _encode_node(node):
    attr = b"".join(dlx._sub(f, payload) for f, payload in node["attr"].items())
    return (dlx._packed_ints(1, node["input_index"]) + dlx._packed_ints(2, node["output_index"]) +
            dlx._sub(3, attr) + dlx._string(5, node["name"]) + dlx._string(6, node["type"]))


def encode_model(model):
    g = model["graph"]
    graph = b"".join(dlx._bytes(1, _encode_node(n)) for n in g["nodes"]) + dlx._string(2, g["name"])
    graph += b"".join(dlx._bytes(3, n.encode()) for n in g["tensor_names"])
    graph += b"".join(dlx._bytes(4, n.encode()) for n in g["output_names"])
    graph += b"".join(dlx._bytes(5, n.encode()) for n in g["input_names"])
    return dlx._sub(1, graph) + dlx._string(2, model["version"]) + dlx._string(3, model["producer_name"])


def _topological(count, inputs_of, rank):
    """Kahn's algorithm over nodes 0..count-1 where inputs_of(i) lists the nodes i reads
    (once per edge) and the ready node of the smallest rank goes first: the std::set<int>
    ready lists of GraphConstructor::Convert and of TopologicalSort in graph.cc."""
    import heapq
    pending = [0] * count
    users = defaultdict(list)
    for i in range(count):
        for src in inputs_of(i):
            users[src].append(i)
            pending[i] += 1
    ready = [(rank[i], i) for i in range(count) if pending[i] == 0]
    heapq.heapify(ready)
    order = []
    while ready:
        _, i = heapq.heappop(ready)
        order.append(i)
        for u in users[i]:
            pending[u] -= 1
            if pending[u] == 0:
                heapq.heappush(ready, (rank[u], u))
    return order


def _producers(nodes):
    producer = {}
    for i, n in enumerate(nodes):
        for t in n["output_index"]:
            producer[t] = i
    return producer


def _sorted_as_constructed(g):
    """The nodes in the order the reference's graph constructor creates them (their ids)."""
    nodes = g["nodes"]
    producer = _producers(nodes)
    for n in nodes:
        for t in n["input_index"]:
            if t not in producer:
                raise ValueError("Node '%s': Unknown input node '%s'" % (
                    n["name"], g["tensor_names"][t] if 0 <= t < len(g["tensor_names"]) else t))
    order = _topological(len(nodes), lambda i: [producer[t] for t in nodes[i]["input_index"]],
                         list(range(len(nodes))))
    if len(order) != len(nodes):
        raise ValueError("the graph has a cycle: %d of %d nodes can be ordered" % (len(order), len(nodes)))
    return [nodes[i] for i in order]


def _emit(g, ids):
    """Graph::ToGraphDef: nodes in topological order by smallest id, isolated nodes that are not
    outputs dropped, tensors renumbered in emission order (a tensor keeps its name)."""
    nodes = g["nodes"]
    producer = _producers(nodes)
    order = _topological(len(nodes), lambda i: [producer[t] for t in nodes[i]["input_index"]], ids)
    if len(order) != len(nodes):
        raise ValueError("the folded graph has a cycle")
    consumed = set(t for n in nodes for t in n["input_index"])
    targets = set(g["output_names"])
    renumber, names, out = {}, [], []
    for i in order:
        n = nodes[i]
        dead = not n["input_index"] and not any(t in consumed for t in n["output_index"])
        if dead and n["name"] not in targets and \
                not any(g["tensor_names"][t] in targets for t in n["output_index"]):
            continue
        for t in n["output_index"]:
            renumber[t] = len(names)
            names.append(g["tensor_names"][t])
        out.append(n)
    for n in out:
        n["input_index"] = [renumber[t] for t in n["input_index"]]
        n["output_index"] = [renumber[t] for t in n["output_index"]]
    g["nodes"], g["tensor_names"] = out, names


def remap(model_bytes):
    """Returns (new model bytes, number of BatchNormalization nodes folded, number of
    activations folded)."""
    model = dlx.decode_model(model_bytes)
    g = model["graph"]
    nodes = g["nodes"] = _sorted_as_constructed(g)
    producer = {}
    consumers = defaultdict(list)
    for i, n in enumerate(nodes):
        for t in n["output_index"]:
            producer[t] = i
        for t in n["input_index"]:
            consumers[t].append(i)
    outputs_kept = set(g["tensor_names"].index(n) for n in g["output_names"] if n in g["tensor_names"])

    def sole_consumer(t, who):
        return consumers[t] == [who] and t not in outputs_kept

    def const_of(t, who):
        i = producer.get(t)
        if i is None or nodes[i]["type"] != "Const" or consumers[t] != [who]:
            return None
        return i

    deleted = set()
    new_consts = []   # Const nodes made by the pass, in the order they were made
    folded_bn = folded_act = 0
    for i in range(len(nodes) - 1, -1, -1):
        if i in deleted:
            continue
        node = nodes[i]
        act = None
        bn_i = i
        if node["type"] in ("Relu", "Clip"):
            src = producer.get(node["input_index"][0])
            if src is None or nodes[src]["type"] != "BatchNormalization" or src in deleted:
                continue
            if not sole_consumer(nodes[src]["output_index"][0], i):
                continue
            act, bn_i = i, src
        elif node["type"] != "BatchNormalization":
            continue
        bn = nodes[bn_i]
        conv_i = producer.get(bn["input_index"][0])
        if conv_i is None or nodes[conv_i]["type"] != "Conv" or conv_i in deleted:
            continue
        conv = nodes[conv_i]
        if not sole_consumer(conv["output_index"][0], bn_i):
            continue
        attr = dlx.decode_conv2d_attr(conv["attr"].get(dlx.ATTR_CONV2D, b""))
        if attr["activation_type"]:
            continue  # already carries an activation: BN cannot move in front of it
        params = [const_of(t, bn_i) for t in bn["input_index"][1:5]]
        w_i = const_of(conv["input_index"][1], conv_i)
        b_i = const_of(conv["input_index"][2], conv_i) if len(conv["input_index"]) > 2 else None
        if None in params or w_i is None or (len(conv["input_index"]) > 2 and b_i is None):
            continue
        gamma, beta, mean, var = (_const_tensor(nodes[p])["float_data"] for p in params)
        eps = np.float32(_decode_floats(bn["attr"].get(dlx.ATTR_BATCHNORM, b""),
                                        {1: "momentum", 2: "epsilon"})["epsilon"])
        wt = _const_tensor(nodes[w_i])
        o = wt["dims"][0]
        if not (gamma.size == beta.size == mean.size == var.size == o):
            continue
        # fp32 arithmetic in the reference's order
        scale = (gamma / np.sqrt(var + eps)).astype(np.float32)
        shift = (-scale * mean + beta).astype(np.float32)
        w = wt["float_data"].reshape(o, -1)
        _set_const(nodes[w_i], wt, (w * scale[:, None]).astype(np.float32))
        if b_i is not None:
            bt = _const_tensor(nodes[b_i])
            _set_const(nodes[b_i], bt, (bt["float_data"] * scale + shift).astype(np.float32))
        else:
            name = "%s:%d" % (conv["name"], len(conv["input_index"]))
            index = len(g["tensor_names"])
            g["tensor_names"].append(name)
            const = dict(name=name, type="Const", input_index=[], output_index=[index], attr={})
            const["attr"][dlx.ATTR_CONST] = dlx._sub(1, dlx.encode_tensor(shift, [o], dlx.ANY, dlx.ANY4))
            new_consts.append(const)
            conv["input_index"].append(index)
        last = nodes[act] if act is not None else bn
        if act is not None:
            attr["activation_type"] = last["type"]
            attr["min"] = 0.0
            attr["max"] = 0.0
            if last["type"] == "Clip":
                attr["max"] = _decode_floats(last["attr"].get(dlx.ATTR_CLIP, b""),
                                             {1: "min", 2: "max"})["max"]
            deleted.add(act)
            folded_act += 1
        conv["attr"][dlx.ATTR_CONV2D] = dlx.encode_conv2d_attr(
            attr["kernel_shape"][0], attr["strides"][0], attr["pads"][0],
            attr["dilations"][0] if attr["dilations"] else 1, attr["group"] or 1,
            attr["activation_type"], attr["min"], attr["max"])
        conv["name"] = last["name"]
        conv["output_index"] = list(last["output_index"])
        deleted.add(bn_i)
        deleted.update(params)
        folded_bn += 1
    # ids: a node of the file keeps its place in construction order, a made constant follows them
    kept = [(i, n) for i, n in enumerate(nodes) if i not in deleted]
    g["nodes"] = [n for _, n in kept] + new_consts
    _emit(g, [i for i, _ in kept] + [len(nodes) + j for j in range(len(new_consts))])
    return encode_model(model), folded_bn, folded_act
