// Reader for the reference's serialized memgraph, so that a graph the reference compiled
// elsewhere can be replayed on this device.
//
// The bytes are what memgraph_t::to_wire writes (src/einsummable/memgraph.cc:258-379): a
// protocol-buffers (proto2) encoding of the message MemGraph of
// src/proto/einsummable.proto:233-238, with MemGraphNode (:216-231), MGApply (:156-165),
// Einsummable (:9-15), Touch (:21-33), Fill (:46-51) and the other MG* messages (:137-214)
// nested in it.  The reference reads them with the generated protobuf classes
// (memgraph_t::from_wire / from_proto, memgraph.cc:381-480); no protobuf compiler or C++
// runtime is assumed here, so the wire format (base-128 varints, tag = field << 3 | type,
// length-delimited sub-messages, repeated scalars packed or not) is decoded by hand.
//
// decode_memgraph gives the node list as data; populate() turns it into an apply graph for
// one device the way the reference's GPU exec graph is made from a memgraph
// (src/engine/gpu/exec_graph.cc:26-245): graph node ids equal memgraph node ids.
#pragma once
#include "exec_graph.h"
#include "ir.h"

#include <cstdint>
#include <optional>
#include <string>
#include <utility>
#include <vector>

namespace es
{

enum class mg_kind : int {
    inputmem = 1,
    inputsto = 2,
    constant = 3,
    apply = 4,
    move = 5,
    evict = 6,
    load = 7,
    partialize = 8,
    alloc = 9,
    del = 10,
    copy = 100,  // the field numbers of MemGraphNode's oneof
};

struct mg_einsummable_t {
    std::vector<uint64_t>         join_shape;
    std::vector<std::vector<int>> inns;
    int                           out_rank = 0;
    std::string                   join;      // scalarop text
    std::string                   castable;  // "" or one of + x v ^
};

struct mg_fill_t {
    bool                  is_lowertri = false;
    std::string           value;  // constant: scalar text
    std::vector<uint64_t> shape;
    std::string           lower, upper;
    // As the reference's reader leaves them: fill_t::from_proto stores the message's ncol
    // in nrow and its nrow in ncol (src/einsummable/fill.cc:137-143), and every consumer
    // downstream sees the swapped pair.  The same is done here.
    uint64_t nrow = 0, ncol = 0;
    int64_t  start = 0;
};

struct mg_node_t {
    mg_kind kind = mg_kind::inputmem;
    int     loc = 0;      // compute location (dst for a move, memory side for evict / load)
    int     src_loc = 0;  // move only
    uint64_t offset = 0, size = 0;  // the node's range (dst for move / copy / load)
    uint64_t src_offset = 0;        // move / copy
    int      storage_loc = 0, storage_id = 0;
    // apply
    std::vector<mem_t>              mems;
    std::optional<mg_einsummable_t> einsummable;
    std::optional<touch_t>          touch;
    int                             group = -1;
    // constant
    mg_fill_t fill;
    std::vector<int> inns;  // ids of the nodes this one waits for, sorted, unique
};

struct memgraph_t {
    int                    num_compute_locs = 0;
    int                    num_storage_locs = 0;
    std::vector<int>       storage_locs;
    std::vector<mg_node_t> nodes;

    // Builds graph nodes for compute location `loc` into an empty apply graph:
    //   inputmem / inputsto / partialize / alloc / del -> dummy (inputsto also declares its
    //   storage slot); apply -> einsummable (scalar variables named in `vars` replaced
    //   first, exec_graph.cc:108-110; a group on an einsummable is an error, :101-103) or
    //   touch with its group; constant -> fill; copy and same-device move -> copy;
    //   evict / load -> host storage.  A node of another location becomes a dummy (the
    //   reference skips those, :88-91); a move between two locations is an error here: one
    //   process drives one device.
    void populate(apply_graph_t& g, int loc,
                  std::vector<std::pair<std::string, double>> const& vars = {}) const;
};

// Throws ir_error on malformed bytes, a missing required field or an unknown node kind
// ("could not parse memgraph", memgraph.cc:384-386).
memgraph_t decode_memgraph(void const* bytes, uint64_t size);

}  // namespace es
