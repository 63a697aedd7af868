// TorchScript boundary: torch.classes.my_classes.DGLGraph and torch.ops.my_ops.*
// with the reference's class layout and operator schemas, so a compiled
// Graphiler plan (a TorchScript graph of my_ops::* nodes) runs unchanged on the
// gfx950 kernels.  This file is host-only glue over the C ABI of
// include/graphiler_amd.h: it owns allocation, argument checks (raised as
// c10::Error, i.e. RuntimeError in Python, like the reference's CHECK_INPUT in
// src/ops/ops.cuh:14-20) and passes the current HIP stream down.
//
// Reference counterparts: include/dglgraph.h:7-75 and src/dglgraph.cpp:5-24
// (class), the `static auto registry` blocks of src/ops/dgl_primitives/spmm.cu:391-406,
// sddmm.cu:131-134, segment_softmax/segment_softmax.cu:27-30,
// segment_mm/segment_mm.cu:35-42 and broadcast/broadcast.cu:102-122 (operators).
#include <torch/custom_class.h>
#include <torch/script.h>

#include <c10/hip/HIPStream.h>

#include <mutex>

#include "../../include/graphiler_amd.h"

namespace {

void check_ga(int code, const char *where) {
  TORCH_CHECK(code == GA_OK, where, ": ", ga_error_string(code), " (code ", code, ")");
}

void check_input(const torch::Tensor &x, const char *name) {
  TORCH_CHECK(x.is_cuda(), name, " must be a CUDA tensor");
  TORCH_CHECK(x.is_contiguous(), name, " must be contiguous");
}

void check_index(const torch::Tensor &x, at::ScalarType t, const char *name) {
  check_input(x, name);
  TORCH_CHECK(x.scalar_type() == t, name, " has the wrong integer type");
}

int feat_dtype(const torch::Tensor &x, const char *name) {
  if (x.scalar_type() == at::kFloat) return GA_F32;
  if (x.scalar_type() == at::kBFloat16) return GA_BF16;
  TORCH_CHECK(false, name, " must be float32 or bfloat16");
  return -1;
}

ga_stream_t current_stream(const torch::Tensor &x) {
  return (ga_stream_t)c10::hip::getCurrentHIPStream(x.device().index()).stream();
}

int64_t feat_dim(const torch::Tensor &x) {
  int64_t d = 1;
  for (int64_t i = 1; i < x.dim(); ++i) d *= x.size(i);
  return d;
}

std::vector<int64_t> out_shape(int64_t rows, const torch::Tensor &x) {
  std::vector<int64_t> shape{rows};
  if (x.dim() > 1)
    for (int64_t i = 1; i < x.dim(); ++i) shape.push_back(x.size(i));
  else
    shape.push_back(1);
  return shape;
}

}  // namespace

// Same public members as the reference's struct; the private part caches what
// the kernels schedule with (slot -> row maps, identity flags, workspace).
struct DGLGraph : torch::CustomClassHolder {
  DGLGraph(torch::Tensor in_pointer, torch::Tensor in_node_indices,
           torch::Tensor in_edge_indices, torch::Tensor out_pointer,
           torch::Tensor out_node_indices, torch::Tensor out_edge_indices,
           torch::Tensor COO_src, torch::Tensor COO_dst,
           at::optional<torch::Tensor> ntype_pointer,
           at::optional<torch::Tensor> etype_pointer)
      : in_pointer(in_pointer), in_node_indices(in_node_indices),
        in_edge_indices(in_edge_indices), out_pointer(out_pointer),
        out_node_indices(out_node_indices), out_edge_indices(out_edge_indices),
        COO_src(COO_src), COO_dst(COO_dst) {
    check_index(in_pointer, at::kInt, "in_pointer");
    check_index(in_node_indices, at::kInt, "in_node_indices");
    check_index(in_edge_indices, at::kInt, "in_edge_indices");
    check_index(out_pointer, at::kInt, "out_pointer");
    check_index(out_node_indices, at::kInt, "out_node_indices");
    check_index(out_edge_indices, at::kInt, "out_edge_indices");
    check_index(COO_src, at::kLong, "COO_src");
    check_index(COO_dst, at::kLong, "COO_dst");
    TORCH_CHECK(in_pointer.size(0) >= 1 && out_pointer.size(0) == in_pointer.size(0),
                "pointers must have num_nodes + 1 entries");
    num_nodes = in_pointer.size(0) - 1;
    num_edges = in_node_indices.size(0);
    TORCH_CHECK(in_edge_indices.size(0) == num_edges &&
                    out_node_indices.size(0) == num_edges &&
                    out_edge_indices.size(0) == num_edges &&
                    COO_src.size(0) == num_edges && COO_dst.size(0) == num_edges,
                "edge columns must all have num_edges entries");
    SetNtypePointer(ntype_pointer);
    SetEtypePointer(etype_pointer);
    // what the kernels schedule with, once, here: the slot -> row maps and whether
    // edge ids are slot numbers (a device-to-host read: not something an operator
    // call should wait for)
    if (in_pointer.is_cuda()) {
      side(false);
      side(true);
    }
  }
  void SetNtypePointer(at::optional<torch::Tensor> pointer) {
    if (pointer.has_value()) check_index(pointer.value(), at::kInt, "ntype_pointer");
    ntype_pointer = pointer;
    num_ntypes = pointer.has_value() ? pointer.value().size(0) - 1 : 1;
  }
  void SetEtypePointer(at::optional<torch::Tensor> pointer) {
    if (pointer.has_value()) check_index(pointer.value(), at::kInt, "etype_pointer");
    std::lock_guard<std::mutex> lock(mu_);
    etype_pointer = pointer;
    num_etypes = pointer.has_value() ? pointer.value().size(0) - 1 : 1;
    // the layouts prepared from the edge types belong to the old pointer
    tiles_ = TypedTiles();
    pairs_ = RelationPairs();
  }
  void SetNtypeCOO(torch::Tensor column) {
    check_index(column, at::kLong, "ntype_COO");
    TORCH_CHECK(column.size(0) == num_nodes, "ntype_COO must have one entry per node");
    ntype_COO = column;
  }
  void SetEtypeCOO(torch::Tensor column) {
    check_index(column, at::kLong, "etype_COO");
    TORCH_CHECK(column.size(0) == num_edges, "etype_COO must have one entry per edge");
    etype_COO = column;
  }

  int64_t num_nodes, num_edges, num_ntypes, num_etypes;
  torch::Tensor in_pointer, in_node_indices, in_edge_indices;
  torch::Tensor out_pointer, out_node_indices, out_edge_indices;
  torch::Tensor COO_src, COO_dst;
  at::optional<torch::Tensor> ntype_pointer, etype_pointer, ntype_COO, etype_COO;

  // ---- derived, built on first use ----------------------------------------
  struct Side {
    torch::Tensor rows;
    bool identity = false;
    bool ready = false;
    int64_t max_degree = 0;     // largest row of this adjacency
  };
  Side side(bool reverse) {
    std::lock_guard<std::mutex> lock(mu_);
    Side &s = reverse ? out_side_ : in_side_;
    if (!s.ready) {
      const torch::Tensor &ptr = reverse ? out_pointer : in_pointer;
      const torch::Tensor &eid = reverse ? out_edge_indices : in_edge_indices;
      s.rows = torch::empty({num_edges}, ptr.options());
      check_ga(ga_csr_row_ids(ptr.data_ptr<int>(), num_nodes, num_edges,
                              s.rows.data_ptr<int>(), current_stream(ptr)),
               "ga_csr_row_ids");
      s.identity = num_edges == 0 ||
                   torch::equal(eid, torch::arange(num_edges, eid.options()));
      s.max_degree = num_nodes > 0 ? (ptr.slice(0, 1) - ptr.slice(0, 0, num_nodes)).max().item<int64_t>() : 0;
      s.ready = true;
    }
    return s;
  }
  // The (destination tile, relation) order of the in-edges that the one-pass typed
  // neighbour sum walks (ga_typed_tiles_build): built on first use, kept with the graph.
  struct TypedTiles {
    torch::Tensor tile_chunk_pointer, chunk_type, slot_src, slot_dst, slot_edge;
    int64_t tile_rows = 128;
    bool ready = false;
  };
  // Returned by value (tensor handles are reference counted): a SetEtypePointer that
  // runs while an operator still uses the layout drops the graph's copy, not the
  // operator's.  Setters must still not run concurrently with operators on one graph
  // object: the operator would read the counts and the type pointer of two states.
  TypedTiles typed_tiles() {
    const Side in = side(false);
    std::lock_guard<std::mutex> lock(mu_);
    if (!tiles_.ready) {
      TORCH_CHECK(etype_pointer.has_value(), "the graph has no edge type pointer");
      const int64_t rows = ga_typed_tile_rows(num_nodes);
      const int64_t cap = ga_typed_tiles_chunk_capacity(num_nodes, num_edges, num_etypes, rows);
      const int64_t tiles = (num_nodes + rows - 1) / rows;
      tiles_.tile_rows = rows;
      const auto i32 = in_pointer.options();
      tiles_.tile_chunk_pointer = torch::empty({tiles + 1}, i32);
      tiles_.chunk_type = torch::empty({std::max<int64_t>(cap, 1)}, i32);
      tiles_.slot_src = torch::empty({std::max<int64_t>(16 * cap, 1)}, i32);
      tiles_.slot_dst = torch::empty({std::max<int64_t>(16 * cap, 4)}, i32.dtype(at::kByte));
      tiles_.slot_edge = torch::empty({std::max<int64_t>(16 * cap, 4)}, i32);
      const size_t bytes = ga_typed_tiles_workspace_bytes(num_nodes, num_edges, num_etypes, rows);
      TORCH_CHECK(bytes > 0, "graph too large for the typed tile layout");
      torch::Tensor ws = torch::empty({(int64_t)bytes}, i32.dtype(at::kByte));
      check_ga(ga_typed_tiles_build(
                   in.rows.data_ptr<int>(), in_node_indices.data_ptr<int>(),
                   in.identity ? nullptr : in_edge_indices.data_ptr<int>(),
                   etype_pointer.value().data_ptr<int>(), num_nodes, num_edges, num_etypes, rows,
                   tiles_.tile_chunk_pointer.data_ptr<int>(), tiles_.chunk_type.data_ptr<int>(),
                   tiles_.slot_src.data_ptr<int>(), tiles_.slot_dst.data_ptr<uint8_t>(),
                   tiles_.slot_edge.data_ptr<int>(), ws.data_ptr(), bytes,
                   current_stream(in_pointer)),
               "ga_typed_tiles_build");
      tiles_.ready = true;
    }
    return tiles_;
  }
  // The (destination, relation) pairs of the in-adjacency: runs of slots with one
  // destination and one relation (the slots of a destination are grouped by relation
  // when edge ids are sorted by type).  Pairs are numbered in slot order; `by_type`
  // lists them by relation, the row order of the typed products.  Built on first use
  // with library sorts and scans; `valid` is false when the slots are not so grouped.
  struct RelationPairs {
    int64_t num_pairs = 0;
    torch::Tensor pair_pointer, pair_of_slot, pair_dst, dst_pointer, type_pointer;   // int32
    torch::Tensor by_type, dst_by_type;                                              // int64
    torch::Tensor rank, rank_of_slot;                                                // int32
    bool valid = false;
    bool ready = false;
  };
  RelationPairs relation_pairs() {   // by value, like typed_tiles()
    const Side in = side(false);
    std::lock_guard<std::mutex> lock(mu_);
    if (!pairs_.ready) {
      pairs_.ready = true;
      if (etype_pointer.has_value() && num_edges > 0) {
        const auto i64 = in_pointer.options().dtype(at::kLong);
        torch::Tensor rows = in.rows.to(at::kLong), eid = in_edge_indices.to(at::kLong);
        torch::Tensor bounds = etype_pointer.value().slice(0, 1).to(at::kLong).contiguous();
        torch::Tensor etype = torch::bucketize(eid, bounds, /*out_int32=*/false, /*right=*/true);
        torch::Tensor key = rows * num_etypes + etype;
        const bool grouped =
            num_edges < 2 || key.slice(0, 1).ge(key.slice(0, 0, num_edges - 1)).all().item<bool>();
        if (grouped) {
          torch::Tensor first = torch::ones({num_edges}, i64.dtype(at::kBool));
          if (num_edges > 1)
            first.slice(0, 1).copy_(key.slice(0, 1).ne(key.slice(0, 0, num_edges - 1)));
          torch::Tensor pair_of_slot = torch::cumsum(first, 0) - 1;
          torch::Tensor starts = torch::nonzero(first).reshape({-1});
          const int64_t P = starts.size(0);
          torch::Tensor pair_key = key.index_select(0, starts);
          torch::Tensor pair_dst = torch::floor_divide(pair_key, num_etypes);
          torch::Tensor pair_type = pair_key - pair_dst * num_etypes;
          torch::Tensor by_type = torch::argsort(pair_type, /*stable=*/true, 0, false);
          torch::Tensor rank = torch::empty_like(by_type);
          rank.index_copy_(0, by_type, torch::arange(P, i64));
          pairs_.num_pairs = P;
          pairs_.pair_pointer =
              torch::cat({starts, torch::full({1}, num_edges, i64)}).to(at::kInt).contiguous();
          pairs_.pair_of_slot = pair_of_slot.to(at::kInt).contiguous();
          pairs_.pair_dst = pair_dst.to(at::kInt).contiguous();
          pairs_.dst_pointer = torch::searchsorted(pair_dst.contiguous(),
                                                   torch::arange(num_nodes + 1, i64))
                                   .to(at::kInt).contiguous();
          pairs_.type_pointer =
              torch::searchsorted(pair_type.index_select(0, by_type).contiguous(),
                                  torch::arange(num_etypes + 1, i64))
                  .to(at::kInt).contiguous();
          pairs_.by_type = by_type.contiguous();
          pairs_.dst_by_type = pair_dst.index_select(0, by_type).contiguous();
          pairs_.rank = rank.to(at::kInt).contiguous();
          pairs_.rank_of_slot = rank.index_select(0, pair_of_slot).to(at::kInt).contiguous();
          pairs_.valid = true;
        }
      }
    }
    return pairs_;
  }
  // Scratch shared by the operators called on this graph: calls that use it must be
  // ordered on one stream (two streams working on one graph object race on it).  It
  // grows on demand; a buffer that was handed out is never freed while the graph
  // lives, because a recorded HIP graph may still replay launches that write to it.
  torch::Tensor workspace(size_t bytes) {
    std::lock_guard<std::mutex> lock(mu_);
    if (!ws_.defined() || (size_t)ws_.numel() < bytes) {
      if (ws_.defined()) retired_ws_.push_back(ws_);
      ws_ = torch::empty({(int64_t)std::max<size_t>(bytes, 256)},
                         in_pointer.options().dtype(at::kByte));
    }
    return ws_;
  }

 private:
  std::mutex mu_;
  Side in_side_, out_side_;
  TypedTiles tiles_;
  RelationPairs pairs_;
  torch::Tensor ws_;
  std::vector<torch::Tensor> retired_ws_;
};

using GraphPtr = c10::intrusive_ptr<DGLGraph>;

namespace {

// edge_rows: u is per-edge in edge-id order and is read through the edge-id
// column in place of the neighbour column (u[e] op w[e])
torch::Tensor spmm(const GraphPtr &g, int op, int reduce, const torch::Tensor &u,
                   const at::optional<torch::Tensor> &w, bool reverse,
                   bool edge_rows = false) {
  check_input(u, "features");
  const int dt = feat_dtype(u, "features");
  const auto &side = g->side(reverse);
  const torch::Tensor &ptr = reverse ? g->out_pointer : g->in_pointer;
  const torch::Tensor &eid = reverse ? g->out_edge_indices : g->in_edge_indices;
  const torch::Tensor &nbr =
      edge_rows ? eid : reverse ? g->out_node_indices : g->in_node_indices;
  const int64_t feat = feat_dim(u);
  int64_t heads = 1;
  if (op >= GA_U_MUL_E) {
    TORCH_CHECK(w.has_value(), "edge weights are required");
    check_input(w.value(), "edge weights");
    TORCH_CHECK(w.value().scalar_type() == at::kFloat, "edge weights must be float32");
    TORCH_CHECK(w.value().size(0) == g->num_edges, "edge weights must have one row per edge");
    heads = feat_dim(w.value());
    TORCH_CHECK(heads > 0 && feat % heads == 0,
                "feature width is not a multiple of the heads");
  }
  TORCH_CHECK(u.size(0) == (op == GA_COPY_E || edge_rows ? g->num_edges : g->num_nodes),
              "features have the wrong number of rows");
  torch::Tensor out = torch::empty(out_shape(g->num_nodes, u), u.options());
  const size_t ws_bytes = ga_spmm_workspace_bytes(g->num_edges, feat);
  torch::Tensor ws = g->workspace(ws_bytes);
  check_ga(ga_spmm_csr(ptr.data_ptr<int>(), side.rows.data_ptr<int>(),
                       nbr.data_ptr<int>(),
                       side.identity ? nullptr : eid.data_ptr<int>(), u.data_ptr(),
                       w.has_value() ? w.value().data_ptr<float>() : nullptr,
                       out.data_ptr(), g->num_nodes, g->num_edges, feat, heads, op,
                       reduce, dt, ws.data_ptr(), (size_t)ws.numel(),
                       current_stream(u)),
           "ga_spmm_csr");
  return out;
}

// spmm.cu:359-373
torch::Tensor SpMMEdge(torch::Tensor features, std::vector<int64_t> dims,
                       bool keep_dim, at::optional<int64_t> dtype,
                       const GraphPtr &graph) {
  return spmm(graph, GA_COPY_E, GA_SUM, features, at::nullopt, false);
}
// spmm.cu:375-389
torch::Tensor SpMMSrc(torch::Tensor features, std::vector<int64_t> dims,
                      bool keep_dim, at::optional<int64_t> dtype,
                      const GraphPtr &graph) {
  return spmm(graph, GA_COPY_U, GA_SUM, features, at::nullopt, false);
}
// act(SpMMSrc | SpMMEdge (features) * row_scale): the sum with the row-wise tail of a
// GCN layer (examples/GCN/GCN.py:26 `torch.relu(torch.sum(mailbox, 1))`, optionally a
// destination-side norm in between) applied where the sums are stored.  activation:
// ga_activation.  The kernel takes a factor that is one fp32 number per row, shaped to
// broadcast over the row ((N, 1) for (N, F) features), on fp32 features; any other
// factor is multiplied afterwards with torch's own broadcasting and promotion, and so
// is the tail of a small sum whose width neither kernel takes at no cost.
torch::Tensor SpMMScaled(torch::Tensor features, at::optional<torch::Tensor> row_scale,
                         int64_t activation, bool edge_rows, const GraphPtr &graph) {
  TORCH_CHECK(activation >= GA_ACT_NONE && activation <= GA_ACT_ELU, "unknown activation");
  check_input(features, "features");
  const int dt = feat_dtype(features, "features");
  const int64_t n = graph->num_nodes;
  bool per_row = false;
  if (row_scale.has_value()) {
    const torch::Tensor &f = row_scale.value();
    per_row = f.is_cuda() && f.scalar_type() == at::kFloat && dt == GA_F32 &&
              f.dim() == std::max<int64_t>(features.dim(), 2) && f.size(0) == n && f.numel() == n;
  }
  // the tail is free on the lanes-per-slot kernel (up to four features; five to seven on
  // graphs of up to 300,000 edges) and cheap for rows that 16-byte accesses tile; for a
  // small result of any other width the sum alone plus two short elementwise kernels is
  // the faster route (measured at 19,717 nodes x 9 features)
  const int64_t width = feat_dim(features);
  const int64_t row_bytes = width * features.element_size();
  const bool on_slots = width <= 4 || (width <= 7 && graph->num_edges <= 300000);
  const bool tail_pays = on_slots || row_bytes % 16 == 0 || n * row_bytes >= (int64_t(8) << 20);
  const bool has_tail = row_scale.has_value() || activation != GA_ACT_NONE;
  if ((row_scale.has_value() && !per_row) || (has_tail && !tail_pays)) {
    torch::Tensor out = spmm(graph, edge_rows ? GA_COPY_E : GA_COPY_U, GA_SUM, features, at::nullopt, false);
    if (row_scale.has_value()) out = out * row_scale.value();
    return activation == GA_ACT_RELU ? at::relu(out) : activation == GA_ACT_ELU ? at::elu(out) : out;
  }
  TORCH_CHECK(features.size(0) == (edge_rows ? graph->num_edges : n),
              "features have the wrong number of rows");
  const auto &side = graph->side(false);
  const int64_t feat = feat_dim(features);
  torch::Tensor factor;
  if (per_row) factor = row_scale.value().contiguous();
  torch::Tensor out = torch::empty(out_shape(n, features), features.options());
  torch::Tensor ws = graph->workspace(ga_spmm_scaled_workspace_bytes(graph->num_edges, feat));
  check_ga(ga_spmm_csr_scaled(
               graph->in_pointer.data_ptr<int>(), side.rows.data_ptr<int>(),
               graph->in_node_indices.data_ptr<int>(),
               side.identity ? nullptr : graph->in_edge_indices.data_ptr<int>(),
               features.data_ptr(), out.data_ptr(), per_row ? factor.data_ptr<float>() : nullptr,
               (int)activation, n, graph->num_edges, feat, edge_rows ? GA_COPY_E : GA_COPY_U, dt,
               ws.data_ptr(), (size_t)ws.numel(), current_stream(features)),
           "ga_spmm_csr_scaled");
  return out;
}
// spmm.cu:286-320
torch::Tensor src_mul_e_sum(torch::Tensor ufeature, torch::Tensor efeature,
                            std::vector<int64_t> dims, bool keep_dim,
                            at::optional<int64_t> dtype,
                            const GraphPtr &graph) {
  return spmm(graph, GA_U_MUL_E, GA_SUM, ufeature, efeature, false);
}
// spmm.cu:322-356
torch::Tensor dst_mul_e_sum(torch::Tensor ufeature, torch::Tensor efeature,
                            std::vector<int64_t> dims, bool keep_dim,
                            at::optional<int64_t> dtype,
                            const GraphPtr &graph) {
  return spmm(graph, GA_U_MUL_E, GA_SUM, ufeature, efeature, true);
}
// generic reducer entry (spmm.cuh:30-71 with functor.cuh:125-213)
torch::Tensor gspmm(torch::Tensor ufeature, at::optional<torch::Tensor> efeature,
                    std::string op, std::string reduce, const GraphPtr &graph) {
  int o = op == "copy_u" ? GA_COPY_U : op == "copy_e" ? GA_COPY_E
          : op == "u_mul_e" ? GA_U_MUL_E : op == "u_add_e" ? GA_U_ADD_E
          : op == "u_sub_e" ? GA_U_SUB_E : op == "u_div_e" ? GA_U_DIV_E : -1;
  int r = reduce == "sum" ? GA_SUM : reduce == "max" ? GA_MAX
          : reduce == "min" ? GA_MIN : -1;
  TORCH_CHECK(o >= 0, "Unsupported SpMM binary operator: ", op);
  TORCH_CHECK(r >= 0, "Unsupported SpMM reducer: ", reduce);
  return spmm(graph, o, r, ufeature, efeature, false);
}

// ---- operands whose feature shapes broadcast -----------------------------------
// UseBcast / CalcBcastOff (bcast.cc:6-71): dimension 0 (nodes or edges) never takes
// part; the others are aligned at the right.  For every element of the flattened
// per-row output, the element of the left and of the right operand that feeds it;
// for the dot product the last dimension is the reduction length and offsets count
// vectors of that length.
struct BcastTables {
  bool use = false;
  int64_t lhs_len = 1, rhs_len = 1, out_len = 1, reduce_size = 1;
  std::vector<int64_t> lhs_off{0}, rhs_off{0}, feat_shape;
};
BcastTables bcast_tables(int op, at::IntArrayRef ls, at::IntArrayRef rs) {
  BcastTables b;
  const int64_t l_nd = ls.size(), r_nd = rs.size();
  for (int64_t i = 1; i < l_nd; ++i) b.lhs_len *= ls[i];
  for (int64_t i = 1; i < r_nd; ++i) b.rhs_len *= rs[i];
  const bool copy = op == GA_BCAST_COPY_LHS || op == GA_BCAST_COPY_RHS;
  if (!copy) {
    b.use = l_nd != r_nd;
    for (int64_t i = 1; !b.use && i < l_nd; ++i) b.use = ls[i] != rs[i];
  }
  const bool dot = op == GA_BCAST_DOT;
  if (dot) {
    TORCH_CHECK(l_nd >= 2 && ls[l_nd - 1] > 0, "dot needs a last dimension to sum over");
    b.reduce_size = ls[l_nd - 1];
  }
  if (!b.use) {
    const at::IntArrayRef &from = op == GA_BCAST_COPY_RHS ? rs : ls;
    b.out_len = (op == GA_BCAST_COPY_RHS ? b.rhs_len : b.lhs_len) / b.reduce_size;
    b.feat_shape.assign(from.begin() + 1, from.end() - (dot ? 1 : 0));
    return b;
  }
  int64_t stride_l = 1, stride_r = 1;
  for (int64_t j = dot ? 1 : 0; j < std::max(l_nd, r_nd) - 1; ++j) {
    const int64_t dl = l_nd - 1 - j < 1 ? 1 : ls[l_nd - 1 - j];
    const int64_t dr = r_nd - 1 - j < 1 ? 1 : rs[r_nd - 1 - j];
    TORCH_CHECK(dl == dr || dl == 1 || dr == 1, "feature shapes do not broadcast");
    const int64_t steps = std::max(dl, dr), inner = b.lhs_off.size();
    std::vector<int64_t> lo(steps * inner), ro(steps * inner);
    for (int64_t s = 0; s < steps; ++s)
      for (int64_t i = 0; i < inner; ++i) {
        lo[s * inner + i] = b.lhs_off[i] + (s < dl ? s : 0) * stride_l;
        ro[s * inner + i] = b.rhs_off[i] + (s < dr ? s : 0) * stride_r;
      }
    b.lhs_off.swap(lo);
    b.rhs_off.swap(ro);
    b.feat_shape.insert(b.feat_shape.begin(), steps);
    b.out_len *= steps;
    stride_l *= dl;
    stride_r *= dr;
  }
  return b;
}
int bcast_op(const std::string &op) {
  return op == "add" ? GA_BCAST_ADD : op == "sub" ? GA_BCAST_SUB : op == "mul" ? GA_BCAST_MUL
         : op == "div" ? GA_BCAST_DIV : op == "copy_lhs" ? GA_BCAST_COPY_LHS
         : op == "copy_rhs" ? GA_BCAST_COPY_RHS : op == "dot" ? GA_BCAST_DOT : -1;
}
torch::Tensor offsets_on(const std::vector<int64_t> &table, const torch::Tensor &like) {
  return torch::tensor(table, at::kLong).to(like.device());
}

// The reference's general SpMM (SpMMCsrKernel with UseBcast, spmm.cuh:30-71):
// out[v] = reduce over the in-edges (out-edges with `reverse`) of op(u[src], e[edge])
// with feature shapes that broadcast; op add | sub | mul | div | copy_lhs | copy_rhs,
// the operand a copy does not read may be None.  fp32, the general (untuned) kernel.
torch::Tensor gspmm_bcast(at::optional<torch::Tensor> u, at::optional<torch::Tensor> e,
                          std::string op, std::string reduce, bool reverse,
                          const GraphPtr &g) {
  const int code = bcast_op(op);
  TORCH_CHECK(code >= 0 && code != GA_BCAST_DOT, "Unsupported SpMM binary operator: ", op);
  const int r = reduce == "sum" ? GA_SUM : reduce == "max" ? GA_MAX : reduce == "min" ? GA_MIN : -1;
  TORCH_CHECK(r >= 0, "Unsupported SpMM reducer: ", reduce);
  const bool use_u = code != GA_BCAST_COPY_RHS, use_e = code != GA_BCAST_COPY_LHS;
  TORCH_CHECK(!use_u || u.has_value(), "node features are required");
  TORCH_CHECK(!use_e || e.has_value(), "edge features are required");
  if (use_u) {
    check_input(u.value(), "u");
    TORCH_CHECK(u.value().scalar_type() == at::kFloat, "the general SpMM is float32 only");
    TORCH_CHECK(u.value().size(0) == g->num_nodes, "u has the wrong number of rows");
  }
  if (use_e) {
    check_input(e.value(), "e");
    TORCH_CHECK(e.value().scalar_type() == at::kFloat, "the general SpMM is float32 only");
    TORCH_CHECK(e.value().size(0) == g->num_edges, "e must have one row per edge");
  }
  const torch::Tensor &ref = use_u ? u.value() : e.value();
  std::vector<int64_t> ls = use_u ? u.value().sizes().vec() : e.value().sizes().vec();
  std::vector<int64_t> rs = use_e ? e.value().sizes().vec() : u.value().sizes().vec();
  const BcastTables b = bcast_tables(code, ls, rs);
  std::vector<int64_t> shape{g->num_nodes};
  shape.insert(shape.end(), b.feat_shape.begin(), b.feat_shape.end());
  torch::Tensor out = torch::empty(shape, ref.options());
  torch::Tensor u_off, e_off;
  if (b.use) {
    u_off = offsets_on(b.lhs_off, ref);
    e_off = offsets_on(b.rhs_off, ref);
  }
  const auto &side = g->side(reverse);
  const torch::Tensor &ptr = reverse ? g->out_pointer : g->in_pointer;
  const torch::Tensor &nbr = reverse ? g->out_node_indices : g->in_node_indices;
  const torch::Tensor &eid = reverse ? g->out_edge_indices : g->in_edge_indices;
  check_ga(ga_spmm_csr_bcast(ptr.data_ptr<int>(), nbr.data_ptr<int>(),
                             side.identity ? nullptr : eid.data_ptr<int>(),
                             use_u ? u.value().data_ptr<float>() : nullptr,
                             use_e ? e.value().data_ptr<float>() : nullptr, out.data_ptr<float>(),
                             nullptr, nullptr, g->num_nodes, g->num_edges,
                             b.use ? u_off.data_ptr<int64_t>() : nullptr,
                             b.use ? e_off.data_ptr<int64_t>() : nullptr,
                             std::max<int64_t>(b.lhs_len, 1), std::max<int64_t>(b.rhs_len, 1),
                             b.out_len, code, r,
                             current_stream(ref)),
           "ga_spmm_csr_bcast");
  return out;
}

// The reference's general SDDMM (sddmm.cuh:34-120): out[e] = op(lhs[id_l(e)], rhs[id_r(e)])
// in edge-id order, each operand on the source nodes ("u"), the edges ("e") or the
// destination nodes ("v") (selector.h:30-60), feature shapes that broadcast; "dot" sums
// the products over the last dimension.  fp32, the general (untuned) kernel.
torch::Tensor gsddmm(torch::Tensor lhs, torch::Tensor rhs, std::string op,
                     std::string lhs_target, std::string rhs_target, const GraphPtr &g) {
  const int code = bcast_op(op);
  TORCH_CHECK(code >= 0, "Unsupported SDDMM binary operator: ", op);
  check_input(lhs, "lhs");
  check_input(rhs, "rhs");
  TORCH_CHECK(lhs.scalar_type() == at::kFloat && rhs.scalar_type() == at::kFloat,
              "the general SDDMM is float32 only");
  auto target = [&](const std::string &t, const torch::Tensor &x, const char *name) {
    const int k = t == "u" ? 0 : t == "e" ? 1 : t == "v" ? 2 : -1;
    TORCH_CHECK(k >= 0, "targets are 'u' (source), 'e' (edge) or 'v' (destination)");
    TORCH_CHECK(x.dim() >= 1 && x.size(0) == (k == 1 ? g->num_edges : g->num_nodes), name,
                " has the wrong number of rows for target '", t, "'");
    return k;
  };
  const int lt = target(lhs_target, lhs, "lhs"), rt = target(rhs_target, rhs, "rhs");
  TORCH_CHECK(code != GA_BCAST_DOT ||
                  (lhs.dim() >= 2 && rhs.dim() >= 2 && lhs.size(-1) == rhs.size(-1)),
              "dot needs operands with the same last dimension");
  const BcastTables b = bcast_tables(code, lhs.sizes(), rhs.sizes());
  std::vector<int64_t> shape{g->num_edges};
  shape.insert(shape.end(), b.feat_shape.begin(), b.feat_shape.end());
  if (shape.size() == 1) shape.push_back(1);
  torch::Tensor out = torch::empty(shape, lhs.options());
  torch::Tensor l_off, r_off;
  if (b.use) {
    l_off = offsets_on(b.lhs_off, lhs);
    r_off = offsets_on(b.rhs_off, lhs);
  }
  check_ga(ga_sddmm_bcast(g->COO_src.data_ptr<int64_t>(), g->COO_dst.data_ptr<int64_t>(),
                          lhs.data_ptr<float>(), rhs.data_ptr<float>(), out.data_ptr<float>(),
                          g->num_edges, lt, rt, b.use ? l_off.data_ptr<int64_t>() : nullptr,
                          b.use ? r_off.data_ptr<int64_t>() : nullptr,
                          std::max<int64_t>(b.lhs_len, 1), std::max<int64_t>(b.rhs_len, 1),
                          b.out_len, b.reduce_size, code, current_stream(out)),
           "ga_sddmm_bcast");
  return out;
}

// SpMMEdge(x * y) for two per-edge operands without the product tensor: one of
// them must be a per-edge / per-head fp32 weight; otherwise multiply, then copy_e
torch::Tensor e_mul_e_sum(torch::Tensor x, torch::Tensor y, const GraphPtr &graph) {
  for (int pass = 0; pass < 2; ++pass) {
    const torch::Tensor &a = pass ? y : x, &b = pass ? x : y;
    if (b.scalar_type() != at::kFloat || a.dim() < 2 || a.size(0) != b.size(0)) continue;
    const bool scalar = b.dim() <= 2 && feat_dim(b) == 1;
    bool per_head = b.dim() == a.dim() && a.dim() >= 3 && b.size(b.dim() - 1) == 1;
    for (int64_t d = 0; per_head && d + 1 < a.dim(); ++d) per_head = a.size(d) == b.size(d);
    if (scalar || per_head) return spmm(graph, GA_U_MUL_E, GA_SUM, a, b, false, true);
  }
  return spmm(graph, GA_COPY_E, GA_SUM, (x * y).contiguous(), at::nullopt, false);
}

struct EdgeColumns {
  const void *lhs, *rhs;
  int bits;
};
EdgeColumns edge_columns(const GraphPtr &g) {
  const auto &side = g->side(false);
  if (side.identity)
    return {g->in_node_indices.data_ptr<int>(), side.rows.data_ptr<int>(), 32};
  return {g->COO_src.data_ptr<int64_t>(), g->COO_dst.data_ptr<int64_t>(), 64};
}

// sddmm.cu:118-129 (alpha accepted and ignored, as there)
torch::Tensor u_add_v_mul_alpha(torch::Tensor src_feature, torch::Tensor dst_feature,
                                int64_t alpha, const GraphPtr &graph) {
  check_input(src_feature, "src_feature");
  check_input(dst_feature, "dst_feature");
  const int dt = feat_dtype(src_feature, "src_feature");
  TORCH_CHECK(dst_feature.scalar_type() == src_feature.scalar_type(),
              "src_feature and dst_feature must share a dtype");
  const int64_t feat = feat_dim(src_feature);
  TORCH_CHECK(feat_dim(dst_feature) == feat,
              "src_feature and dst_feature must share a width");
  torch::Tensor out = torch::empty(out_shape(graph->num_edges, src_feature),
                                   src_feature.options().dtype(at::kFloat));
  // two or four fp32 values per node on a graph stored by destination: walk the
  // adjacency (rows from the row pointer, one index column instead of two)
  if (dt == GA_F32 && (feat == 2 || feat == 4) && graph->num_edges > 0 &&
      graph->side(false).identity) {
    const int rc = ga_sddmm_u_op_v_adj(
        graph->in_pointer.data_ptr<int>(), graph->side(false).rows.data_ptr<int>(),
        graph->in_node_indices.data_ptr<int>(), src_feature.data_ptr<float>(),
        dst_feature.data_ptr<float>(), out.data_ptr<float>(), graph->num_nodes,
        graph->num_edges, feat, GA_SDDMM_ADD, current_stream(out));
    if (rc != GA_EALIGN && rc != GA_EUNSUPPORTED) {
      check_ga(rc, "ga_sddmm_u_op_v_adj");
      return out;
    }
  }
  const EdgeColumns c = edge_columns(graph);
  check_ga(ga_sddmm_u_add_v(c.lhs, c.rhs, c.bits, src_feature.data_ptr(),
                            dst_feature.data_ptr(), out.data_ptr<float>(),
                            graph->num_edges, feat, dt, current_stream(out)),
           "ga_sddmm_u_add_v");
  return out;
}

// functor.cuh:103-116 + sddmm.cuh:80-120 (never registered by the reference)
torch::Tensor u_dot_v(torch::Tensor src_feature, torch::Tensor dst_feature,
                      const GraphPtr &graph) {
  check_input(src_feature, "src_feature");
  check_input(dst_feature, "dst_feature");
  const int dt = feat_dtype(src_feature, "src_feature");
  TORCH_CHECK(dst_feature.scalar_type() == src_feature.scalar_type() &&
                  dst_feature.sizes().slice(1) == src_feature.sizes().slice(1),
              "src_feature and dst_feature must share dtype and shape");
  TORCH_CHECK(src_feature.dim() == 2 || src_feature.dim() == 3,
              "u_dot_v expects (N, D) or (N, H, D) features");
  const int64_t heads = src_feature.dim() == 3 ? src_feature.size(1) : 1;
  const int64_t dim = src_feature.size(src_feature.dim() - 1);
  torch::Tensor out = torch::empty({graph->num_edges, heads},
                                   src_feature.options().dtype(at::kFloat));
  const EdgeColumns c = edge_columns(graph);
  check_ga(ga_sddmm_u_dot_v(c.lhs, c.rhs, c.bits, src_feature.data_ptr(),
                            dst_feature.data_ptr(), out.data_ptr<float>(),
                            graph->num_edges, heads, dim, dt, current_stream(out)),
           "ga_sddmm_u_dot_v");
  return out;
}

// segment_softmax.cu:3-24
torch::Tensor SegmentSoftmaxForward(torch::Tensor features, int64_t dim,
                                    at::optional<int64_t> dtype,
                                    const GraphPtr &graph) {
  check_input(features, "features");
  TORCH_CHECK(dim == 1, "SegmentSoftmax reduces over dim 1 of the mailbox");
  TORCH_CHECK(features.scalar_type() == at::kFloat, "features must be float32");
  TORCH_CHECK(features.size(0) == graph->num_edges, "features must have one row per edge");
  const int64_t heads = feat_dim(features);
  const auto &side = graph->side(false);
  torch::Tensor y = torch::empty_like(features);
  torch::Tensor ws = graph->workspace(ga_softmax_workspace_bytes(graph->num_edges, heads));
  check_ga(ga_segment_softmax(graph->in_pointer.data_ptr<int>(),
                              side.rows.data_ptr<int>(),
                              side.identity ? nullptr
                                            : graph->in_edge_indices.data_ptr<int>(),
                              features.data_ptr<float>(), y.data_ptr<float>(),
                              graph->num_nodes, graph->num_edges, heads,
                              ws.data_ptr(), (size_t)ws.numel(), current_stream(y)),
           "ga_segment_softmax");
  return y;
}

// segment_mm.cu:4-21
torch::Tensor segment_mm(const torch::Tensor &features, const torch::Tensor &weights,
                         const at::optional<torch::Tensor> &type_pointer,
                         int64_t num_types, int64_t rows_expected) {
  check_input(features, "features");
  check_input(weights, "weights");
  const int dt = feat_dtype(features, "features");
  TORCH_CHECK(weights.scalar_type() == features.scalar_type(),
              "features and weights must share a dtype");
  TORCH_CHECK(type_pointer.has_value(), "the graph has no type pointer for this operator");
  TORCH_CHECK(weights.dim() == 3 || weights.dim() == 4,
              "weights must be (T, K, M) or (T, H, K, M)");
  const int64_t heads = weights.dim() == 4 ? weights.size(1) : 1;
  const int64_t K = weights.size(weights.dim() - 2), M = weights.size(weights.dim() - 1);
  TORCH_CHECK(weights.size(0) == num_types, "weights must have one matrix per type");
  const int64_t rows = features.size(0);
  TORCH_CHECK(rows == rows_expected && feat_dim(features) == heads * K,
              "features must be (rows, heads*K)");
  torch::Tensor out = torch::empty({rows, heads * M}, features.options());
  check_ga(ga_segment_mm(type_pointer.value().data_ptr<int>(), num_types,
                         features.data_ptr(), weights.data_ptr(), out.data_ptr(),
                         rows, heads, K, M, dt, current_stream(out)),
           "ga_segment_mm");
  return out;
}
// segment_mm.cu:23-27
torch::Tensor SegmentMMNode(torch::Tensor features, torch::Tensor weights,
                            const GraphPtr &graph) {
  return segment_mm(features, weights, graph->ntype_pointer, graph->num_ntypes,
                    graph->num_nodes);
}
// SegmentMMNode(features, weights) * row_scale with an (N, 1) factor applied to the fp32
// sums before they are rounded: the `trans_out * alpha.unsqueeze(1)` of
// examples/HGT/HGT.py:58-60 without a pass over the result.  Any other factor (another
// shape, a dtype that would promote the product) multiplies the result afterwards.
torch::Tensor SegmentMMNodeScaled(torch::Tensor features, torch::Tensor weights,
                                  torch::Tensor row_scale, const GraphPtr &graph) {
  const bool fits = row_scale.is_cuda() && row_scale.dim() == 2 && row_scale.size(1) == 1 &&
                    row_scale.size(0) == graph->num_nodes && row_scale.is_floating_point() &&
                    features.is_floating_point() && features.dim() == 2 &&
                    features.size(0) == graph->num_nodes && (weights.dim() == 3 || weights.dim() == 4) &&
                    at::promote_types(features.scalar_type(), row_scale.scalar_type()) ==
                        features.scalar_type();
  if (fits) {
    check_input(features, "features");
    check_input(weights, "weights");
    const int dt = feat_dtype(features, "features");
    TORCH_CHECK(weights.scalar_type() == features.scalar_type(),
                "features and weights must share a dtype");
    TORCH_CHECK(graph->ntype_pointer.has_value(), "the graph has no type pointer for this operator");
    const int64_t heads = weights.dim() == 4 ? weights.size(1) : 1;
    const int64_t K = weights.size(weights.dim() - 2), M = weights.size(weights.dim() - 1);
    TORCH_CHECK(weights.size(0) == graph->num_ntypes, "weights must have one matrix per type");
    TORCH_CHECK(feat_dim(features) == heads * K, "features must be (rows, heads*K)");
    torch::Tensor rs = row_scale.to(at::kFloat).contiguous();
    torch::Tensor out = torch::empty({graph->num_nodes, heads * M}, features.options());
    const int rc = ga_segment_mm_gather(
        graph->ntype_pointer.value().data_ptr<int>(), graph->num_ntypes, features.data_ptr(),
        nullptr, weights.data_ptr(), out.data_ptr(), nullptr, nullptr, nullptr, nullptr,
        rs.data_ptr<float>(), graph->num_nodes, heads, K, M, dt, current_stream(out));
    if (rc != GA_EUNSUPPORTED) {
      check_ga(rc, "ga_segment_mm_gather");
      return out;
    }
  }
  return SegmentMMNode(features, weights, graph) * row_scale;
}
torch::Tensor BroadcastNodeType(torch::Tensor features, const GraphPtr &graph);
// SegmentMMNode(features, weights) * g(BroadcastNodeType(gate.unsqueeze(1))) with g the
// sigmoid (or the identity): the output projection of examples/HGT/HGT.py:58-60 with its
// per-node-type gate.  The product's kernel takes the per-type factor where it runs the
// shape (ga_segment_mm_gated: bf16, wide outputs); otherwise the factor is formed per row
// and handed to SegmentMMNodeScaled.
torch::Tensor SegmentMMNodeGated(torch::Tensor features, torch::Tensor weights, torch::Tensor gate,
                                 bool sigmoid, const GraphPtr &graph) {
  TORCH_CHECK(gate.dim() == 1 && gate.size(0) == graph->num_ntypes,
              "gate must have one entry per node type");
  // (a gate that would promote the product, e.g. fp32 on bf16 features, keeps the
  // meaning of the expression: it multiplies the result afterwards, below)
  if (features.is_cuda() && features.scalar_type() == at::kBFloat16 &&
      at::promote_types(features.scalar_type(), gate.scalar_type()) == features.scalar_type() &&
      weights.scalar_type() == at::kBFloat16 && features.dim() == 2 && weights.dim() == 3 &&
      features.size(0) == graph->num_nodes && weights.size(0) == graph->num_ntypes &&
      features.size(1) == weights.size(1) && gate.is_floating_point() &&
      graph->ntype_pointer.has_value()) {
    check_input(features, "features");
    check_input(weights, "weights");
    torch::Tensor g32 = gate.to(at::kFloat).contiguous();
    check_input(g32, "gate");
    torch::Tensor out = torch::empty({graph->num_nodes, weights.size(2)}, features.options());
    const int rc = ga_segment_mm_gated(
        graph->ntype_pointer.value().data_ptr<int>(), graph->num_ntypes, features.data_ptr(),
        weights.data_ptr(), out.data_ptr(), g32.data_ptr<float>(), sigmoid ? 1 : 0,
        graph->num_nodes, weights.size(1), weights.size(2), GA_BF16, current_stream(out));
    if (rc != GA_EUNSUPPORTED) {
      check_ga(rc, "ga_segment_mm_gated");
      return out;
    }
  }
  torch::Tensor factor = sigmoid ? torch::sigmoid(gate) : gate;
  return SegmentMMNodeScaled(features, weights, BroadcastNodeType(factor.unsqueeze(1), graph), graph);
}
// segment_mm.cu:29-33
torch::Tensor SegmentMMEdge(torch::Tensor features, torch::Tensor weights,
                            const GraphPtr &graph) {
  return segment_mm(features, weights, graph->etype_pointer, graph->num_etypes,
                    graph->num_edges);
}

// [SegmentMMNode(features, w, graph) for w in weights] with the rows of `features` read
// once when the weights have one shape (HGT's K, Q, V: examples/HGT/HGT.py:35-44)
std::vector<torch::Tensor> SegmentMMNodeStacked(torch::Tensor features,
                                                std::vector<torch::Tensor> weights,
                                                const GraphPtr &graph) {
  bool same = !weights.empty() && weights.size() <= 4;
  for (const torch::Tensor &w : weights)
    same = same && w.dim() == 3 && w.sizes() == weights[0].sizes() && w.is_cuda() &&
           w.is_contiguous() && w.scalar_type() == features.scalar_type();
  std::vector<torch::Tensor> outs;
  if (!same) {
    for (const torch::Tensor &w : weights) outs.push_back(SegmentMMNode(features, w, graph));
    return outs;
  }
  check_input(features, "features");
  const int dt = feat_dtype(features, "features");
  TORCH_CHECK(graph->ntype_pointer.has_value(), "the graph has no type pointer for this operator");
  const int64_t K = weights[0].size(1), M = weights[0].size(2), rows = features.size(0);
  TORCH_CHECK(weights[0].size(0) == graph->num_ntypes, "weights must have one matrix per type");
  TORCH_CHECK(rows == graph->num_nodes && feat_dim(features) == K, "features must be (rows, K)");
  std::vector<const void *> wp;
  std::vector<void *> yp;
  for (const torch::Tensor &w : weights) {
    outs.push_back(torch::empty({rows, M}, features.options()));
    wp.push_back(w.data_ptr());
    yp.push_back(outs.back().data_ptr());
  }
  check_ga(ga_segment_mm_stacked(graph->ntype_pointer.value().data_ptr<int>(), graph->num_ntypes,
                                 features.data_ptr(), wp.data(), yp.data(), (int64_t)wp.size(),
                                 rows, K, M, dt, current_stream(features)),
           "ga_segment_mm_stacked");
  return outs;
}

torch::Tensor gather(const torch::Tensor &features, const torch::Tensor &index);

struct MmShape { int64_t heads, K, M; int dt; };
MmShape edge_mm_shape(const torch::Tensor &features, const torch::Tensor &weights,
                      const GraphPtr &graph) {
  check_input(features, "features");
  check_input(weights, "weights");
  MmShape s;
  s.dt = feat_dtype(features, "features");
  TORCH_CHECK(weights.scalar_type() == features.scalar_type(),
              "features and weights must share a dtype");
  TORCH_CHECK(graph->etype_pointer.has_value(),
              "the graph has no type pointer for this operator");
  TORCH_CHECK(weights.dim() == 3 || weights.dim() == 4,
              "weights must be (T, K, M) or (T, H, K, M)");
  s.heads = weights.dim() == 4 ? weights.size(1) : 1;
  s.K = weights.size(weights.dim() - 2);
  s.M = weights.size(weights.dim() - 1);
  TORCH_CHECK(weights.size(0) == graph->num_etypes, "weights must have one matrix per type");
  TORCH_CHECK(features.size(0) == graph->num_nodes && feat_dim(features) == s.heads * s.K,
              "features must be (nodes, heads*K)");
  return s;
}
const torch::Tensor &endpoint_column(const GraphPtr &graph, int64_t which) {
  TORCH_CHECK(which == 0 || which == 1, "endpoint must be 0 (source) or 1 (destination)");
  return which == 0 ? graph->COO_src : graph->COO_dst;
}

// broadcast.cu:58-69 + segment_mm.cu:29-33 as one pass:
// out[e] = features[endpoint(e)] @ weights[type(e)]
// row_scale: an (E,) / (E, 1) fp32 tensor multiplies row e of the result (the
// per-edge norm of examples/RGCN/RGCN.py:29); any other shape multiplies the
// result afterwards with ATen's broadcasting
// A factor of `product * factor` that a kernel can apply to its fp32 sums without changing
// what the expression means: one value per row ((rows,) or (rows, 1)) of a floating dtype
// that does not promote the product (bf16 features times an fp32 factor is an fp32 tensor
// in eager PyTorch, and stays one here: such a factor multiplies the result afterwards).
// Returns the factor as contiguous fp32, or an undefined tensor.
torch::Tensor kernel_row_factor(const at::optional<torch::Tensor> &row_scale, int64_t rows,
                                const torch::Tensor &features) {
  if (!row_scale.has_value()) return torch::Tensor();
  const torch::Tensor &r = row_scale.value();
  if (!r.is_cuda() || !r.is_floating_point() || r.numel() != rows || r.dim() < 1 || r.dim() > 2 ||
      r.size(0) != rows ||
      at::promote_types(features.scalar_type(), r.scalar_type()) != features.scalar_type())
    return torch::Tensor();
  return r.to(at::kFloat).contiguous();
}
// The same factor as an operand of `out * factor` (one value per row broadcasts over the row).
torch::Tensor as_row_operand(const torch::Tensor &r, int64_t rows) {
  return r.dim() == 1 && r.size(0) == rows ? r.unsqueeze(1) : r;
}

torch::Tensor SegmentMMEdgeGather(torch::Tensor features, torch::Tensor weights,
                                  int64_t endpoint, at::optional<torch::Tensor> row_scale,
                                  const GraphPtr &graph) {
  const MmShape s = edge_mm_shape(features, weights, graph);
  const torch::Tensor &index = endpoint_column(graph, endpoint);
  torch::Tensor out = torch::empty({graph->num_edges, s.heads * s.M}, features.options());
  const torch::Tensor factor = kernel_row_factor(row_scale, graph->num_edges, features);
  const float *rs = factor.defined() ? factor.data_ptr<float>() : nullptr;
  torch::Tensor late;            // a factor the kernel does not take
  if (row_scale.has_value() && !rs) late = as_row_operand(row_scale.value(), graph->num_edges);
  const int rc = ga_segment_mm_gather(
      graph->etype_pointer.value().data_ptr<int>(), graph->num_etypes, features.data_ptr(),
      index.data_ptr<int64_t>(), weights.data_ptr(), out.data_ptr(), nullptr, nullptr,
      nullptr, nullptr, rs, graph->num_edges, s.heads, s.K, s.M, s.dt, current_stream(out));
  if (rc == GA_EUNSUPPORTED) {     // shape outside the matrix-core tile
    out = segment_mm(gather(features, index), weights, graph->etype_pointer,
                     graph->num_etypes, graph->num_edges);
    if (rs) late = as_row_operand(row_scale.value(), graph->num_edges);
  } else {
    check_ga(rc, "ga_segment_mm_gather");
  }
  return late.defined() ? out * late : out;
}

// SpMMEdge(SegmentMMEdgeGather(features, weights, 0, row_scale)): an RGCN layer's message
// and reduce steps (examples/RGCN/RGCN.py:25-33).  One pass without the per-edge
// messages where that kernel is the faster one (the small products: K * M up to 2048,
// e.g. 16 -> 64 and 64 -> 8), the two operators elsewhere.
torch::Tensor TypedSpMMEdge(torch::Tensor features, torch::Tensor weights,
                            at::optional<torch::Tensor> row_scale, const GraphPtr &graph) {
  const MmShape s = edge_mm_shape(features, weights, graph);
  const torch::Tensor factor = kernel_row_factor(row_scale, graph->num_edges, features);
  const float *rs = factor.defined() ? factor.data_ptr<float>() : nullptr;
  const bool plain_scale = !row_scale.has_value() || rs;
  const bool cols_ok = s.M == 8 || s.M == 16 || s.M == 32 || s.M == 64;
  // fp32: the one pass keeps one accumulator per destination, whose rounding error grows
  // with the in-degree (6e-6 of the sum at 16,000 in-edges of one sign); beyond 8192 the
  // operator pair with its run-wise sums is taken
  const bool accurate = s.dt != GA_F32 || graph->side(false).max_degree <= 8192;
  if (plain_scale && weights.dim() == 3 && features.dim() == 2 && s.K % 16 == 0 && cols_ok &&
      s.K * s.M <= 2048 && accurate) {
    const DGLGraph::TypedTiles &t = graph->typed_tiles();
    torch::Tensor out = torch::empty({graph->num_nodes, s.M}, features.options());
    const int rc = ga_typed_spmm(
        t.tile_chunk_pointer.data_ptr<int>(), t.chunk_type.data_ptr<int>(),
        t.slot_src.data_ptr<int>(), t.slot_dst.data_ptr<uint8_t>(), t.slot_edge.data_ptr<int>(),
        features.data_ptr(), weights.data_ptr(), rs, out.data_ptr(), graph->num_nodes,
        features.size(0), graph->num_edges, graph->num_etypes, t.tile_rows, s.K, s.M, s.dt,
        current_stream(out));
    if (rc != GA_EUNSUPPORTED) {
      check_ga(rc, "ga_typed_spmm");
      return out;
    }
  }
  return spmm(graph, GA_COPY_E, GA_SUM, SegmentMMEdgeGather(features, weights, 0, row_scale, graph),
              at::nullopt, false);
}

// out[e, h] = <features[endpoint(e)] @ weights[type(e)], other[other_endpoint(e)]>
// (examples/HGT/HGT.py:42-45), fp32 (E, heads)
torch::Tensor SegmentMMEdgeDot(torch::Tensor features, torch::Tensor weights,
                               int64_t endpoint, torch::Tensor other,
                               int64_t other_endpoint, at::optional<torch::Tensor> scale,
                               const GraphPtr &graph) {
  const MmShape s = edge_mm_shape(features, weights, graph);
  torch::Tensor sc;      // (T, heads) fp32: out[e, h] *= scale[type(e), h]
  torch::Tensor late;    // a per-type factor of another shape: broadcast afterwards
  if (scale.has_value()) {
    check_input(scale.value(), "scale");
    if (scale.value().numel() == graph->num_etypes * s.heads) {
      sc = scale.value().to(at::kFloat).contiguous();
    } else {
      TORCH_CHECK(graph->etype_COO.has_value(), "the graph has no edge-type column");
      late = gather(scale.value(), graph->etype_COO.value());
    }
  }
  check_input(other, "other");
  TORCH_CHECK(other.scalar_type() == features.scalar_type() &&
                  other.size(0) == graph->num_nodes && feat_dim(other) == s.heads * s.M,
              "other must be (nodes, heads*M) of the features' dtype");
  const torch::Tensor &xi = endpoint_column(graph, endpoint);
  const torch::Tensor &qi = endpoint_column(graph, other_endpoint);
  torch::Tensor out =
      torch::empty({graph->num_edges, s.heads}, features.options().dtype(at::kFloat));
  const int rc = ga_segment_mm_gather(
      graph->etype_pointer.value().data_ptr<int>(), graph->num_etypes, features.data_ptr(),
      xi.data_ptr<int64_t>(), weights.data_ptr(), nullptr, other.data_ptr(),
      qi.data_ptr<int64_t>(), sc.defined() ? sc.data_ptr<float>() : nullptr,
      out.data_ptr<float>(), nullptr, graph->num_edges, s.heads, s.K, s.M, s.dt,
      current_stream(out));
  if (rc == GA_EUNSUPPORTED) {
    torch::Tensor y = SegmentMMEdgeGather(features, weights, endpoint, at::nullopt, graph);
    torch::Tensor q = gather(other, qi).reshape(y.sizes());
    torch::Tensor d = (y.to(at::kFloat) * q.to(at::kFloat))
                          .reshape({graph->num_edges, s.heads, s.M})
                          .sum(-1);
    TORCH_CHECK(!sc.defined() || graph->etype_COO.has_value(),
                "the graph has no edge-type column");
    if (sc.defined())
      d = d * gather(sc.reshape({graph->num_etypes, s.heads}), graph->etype_COO.value());
    return late.defined() ? d * late : d;
  }
  check_ga(rc, "ga_segment_mm_gather");
  return late.defined() ? out * late : out;
}

torch::Tensor gather(const torch::Tensor &features, const torch::Tensor &index) {
  check_input(features, "features");
  std::vector<int64_t> shape{index.size(0)};
  for (int64_t i = 1; i < features.dim(); ++i) shape.push_back(features.size(i));
  torch::Tensor out = torch::empty(shape, features.options());
  check_ga(ga_gather_rows(index.data_ptr(), 64, features.data_ptr(), out.data_ptr(),
                          index.size(0), feat_dim(features) * features.element_size(),
                          current_stream(out)),
           "ga_gather_rows");
  return out;
}
// broadcast.cu:58-100
torch::Tensor BroadcastSrcNode(torch::Tensor features, const GraphPtr &graph) {
  return gather(features, graph->COO_src);
}
torch::Tensor BroadcastDstNode(torch::Tensor features, const GraphPtr &graph) {
  return gather(features, graph->COO_dst);
}
torch::Tensor BroadcastNodeType(torch::Tensor features, const GraphPtr &graph) {
  TORCH_CHECK(graph->ntype_COO.has_value(), "the graph has no node-type column");
  return gather(features, graph->ntype_COO.value());
}
torch::Tensor BroadcastSrcNodeType(torch::Tensor features, const GraphPtr &graph) {
  return BroadcastSrcNode(BroadcastNodeType(features, graph), graph);
}
torch::Tensor BroadcastDstNodeType(torch::Tensor features, const GraphPtr &graph) {
  return BroadcastDstNode(BroadcastNodeType(features, graph), graph);
}
torch::Tensor BroadcastEdgeType(torch::Tensor features, const GraphPtr &graph) {
  TORCH_CHECK(graph->etype_COO.has_value(), "the graph has no edge-type column");
  return gather(features, graph->etype_COO.value());
}
// broadcast.cu:3-9
int64_t get_feat_dim(torch::Tensor features) { return feat_dim(features); }

// fused u_add_v -> leaky_relu -> SegmentSoftmax -> src_mul_e_sum
torch::Tensor gat_aggregate(torch::Tensor el, torch::Tensor er, torch::Tensor z,
                            double negative_slope, const GraphPtr &graph) {
  check_input(el, "el");
  check_input(er, "er");
  check_input(z, "z");
  const int dt = feat_dtype(z, "z");
  // the attention terms of a bf16 plan may arrive as bf16 (mm(z, attn_weight) on the
  // stored z): the logits are formed in fp32 either way
  TORCH_CHECK(el.is_floating_point() && er.is_floating_point(), "el and er must be floating point");
  el = el.to(at::kFloat).contiguous();
  er = er.to(at::kFloat).contiguous();
  const int64_t heads = feat_dim(el), feat = feat_dim(z);
  TORCH_CHECK(feat_dim(er) == heads && heads > 0 && feat % heads == 0,
              "inconsistent head count");
  TORCH_CHECK(el.size(0) == graph->num_nodes && er.size(0) == graph->num_nodes &&
                  z.size(0) == graph->num_nodes, "inputs must have one row per node");
  const auto &side = graph->side(false);
  torch::Tensor out = torch::empty(out_shape(graph->num_nodes, z), z.options());
  torch::Tensor ws = graph->workspace(ga_gat_workspace_bytes(graph->num_edges, feat, heads));
  check_ga(ga_gat_aggregate(graph->in_pointer.data_ptr<int>(),
                            side.rows.data_ptr<int>(),
                            graph->in_node_indices.data_ptr<int>(),
                            el.data_ptr<float>(), er.data_ptr<float>(), z.data_ptr(),
                            out.data_ptr(), graph->num_nodes, graph->num_edges, heads,
                            feat / heads, (float)negative_slope, dt, ws.data_ptr(),
                            (size_t)ws.numel(), current_stream(out)),
           "ga_gat_aggregate");
  return out;
}

// gat_aggregate that may recompute the source term from the gathered rows: with
// a_l (heads * dim elements) at hand, a table of source terms of 16 MB or more
// (it no longer stays cached, and gathering it costs a memory sector per edge)
// is not read at all; smaller tables take the ordinary pass.
torch::Tensor gat_aggregate_al(torch::Tensor a_l, torch::Tensor el, torch::Tensor er,
                               torch::Tensor z, double negative_slope, const GraphPtr &graph) {
  constexpr int64_t kTableLimit = 16 << 20;
  if (el.numel() * 4 < kTableLimit) return gat_aggregate(el, er, z, negative_slope, graph);
  check_input(er, "er");
  check_input(z, "z");
  TORCH_CHECK(a_l.is_cuda(), "a_l must be a CUDA tensor");
  const int dt = feat_dtype(z, "z");
  TORCH_CHECK(er.is_floating_point(), "er must be floating point");
  er = er.to(at::kFloat).contiguous();
  const int64_t heads = feat_dim(er), feat = feat_dim(z);
  TORCH_CHECK(heads > 0 && feat % heads == 0 && a_l.numel() == feat, "inconsistent head count");
  TORCH_CHECK(er.size(0) == graph->num_nodes && z.size(0) == graph->num_nodes,
              "inputs must have one row per node");
  torch::Tensor al = a_l.to(at::kFloat).contiguous();
  const auto &side = graph->side(false);
  torch::Tensor out = torch::empty(out_shape(graph->num_nodes, z), z.options());
  torch::Tensor ws = graph->workspace(ga_gat_workspace_bytes(graph->num_edges, feat, heads));
  const int rc = ga_gat_aggregate_from_z(
      graph->in_pointer.data_ptr<int>(), side.rows.data_ptr<int>(),
      graph->in_node_indices.data_ptr<int>(), al.data_ptr<float>(), er.data_ptr<float>(),
      z.data_ptr(), out.data_ptr(), graph->num_nodes, graph->num_edges, heads, feat / heads,
      (float)negative_slope, dt, ws.data_ptr(), (size_t)ws.numel(), current_stream(out));
  if (rc == GA_EUNSUPPORTED) return gat_aggregate(el, er, z, negative_slope, graph);
  check_ga(rc, "ga_gat_aggregate_from_z");
  return out;
}

// SegmentSoftmax -> mul -> SpMMEdge (examples/HGT/HGT.py:50-53) in one pass:
// out[v] = sum over in-edges e of softmax_v(logits)[e] * messages[e]
torch::Tensor edge_softmax_sum(torch::Tensor logits, torch::Tensor messages,
                               const GraphPtr &graph) {
  check_input(logits, "logits");
  check_input(messages, "messages");
  const int64_t heads = feat_dim(logits), feat = feat_dim(messages);
  const bool fits = logits.scalar_type() == at::kFloat && messages.dim() >= 2 &&
                    heads > 0 && feat % heads == 0 &&
                    (messages.scalar_type() == at::kFloat ||
                     messages.scalar_type() == at::kBFloat16);
  if (!fits)      // the two operators it stands for
    return e_mul_e_sum(SegmentSoftmaxForward(logits, 1, at::nullopt, graph), messages, graph);
  const int dt = feat_dtype(messages, "messages");
  TORCH_CHECK(logits.size(0) == graph->num_edges && messages.size(0) == graph->num_edges,
              "logits and messages must have one row per edge");
  const auto &side = graph->side(false);
  torch::Tensor out = torch::empty(out_shape(graph->num_nodes, messages), messages.options());
  torch::Tensor ws = graph->workspace(ga_gat_workspace_bytes(graph->num_edges, feat, heads));
  check_ga(ga_edge_softmax_sum(graph->in_pointer.data_ptr<int>(), side.rows.data_ptr<int>(),
                               side.identity ? nullptr
                                             : graph->in_edge_indices.data_ptr<int>(),
                               logits.data_ptr<float>(), messages.data_ptr(), out.data_ptr(),
                               graph->num_nodes, graph->num_edges, heads, feat / heads, dt,
                               ws.data_ptr(), (size_t)ws.numel(), current_stream(out)),
           "ga_edge_softmax_sum");
  return out;
}

// out[v] = sum over the in-edges e of v of softmax_v(<k[src], q[v]>)[e] * v[src], per head
// (sum(k * q) -> SegmentSoftmax -> mul -> SpMM in one pass): k, q, v (N, H, D) or (N, D).
torch::Tensor dot_attention_sum(torch::Tensor k, torch::Tensor q, torch::Tensor v,
                                const GraphPtr &graph) {
  check_input(k, "k");
  check_input(q, "q");
  check_input(v, "v");
  const int dt = feat_dtype(k, "k");
  TORCH_CHECK((k.dim() == 2 || k.dim() == 3) && k.sizes() == q.sizes() && k.sizes() == v.sizes() &&
                  q.scalar_type() == k.scalar_type() && v.scalar_type() == k.scalar_type() &&
                  k.size(0) == graph->num_nodes,
              "k, q and v must be (nodes, heads, D) or (nodes, D) of one dtype");
  const int64_t heads = k.dim() == 3 ? k.size(1) : 1, d = k.size(k.dim() - 1);
  const auto &side = graph->side(false);
  torch::Tensor out = torch::empty_like(v);
  torch::Tensor ws = graph->workspace(ga_gat_workspace_bytes(graph->num_edges, heads * d, heads));
  check_ga(ga_dot_attention_sum(graph->in_pointer.data_ptr<int>(), side.rows.data_ptr<int>(),
                                graph->in_node_indices.data_ptr<int>(), side.rows.data_ptr<int>(),
                                k.data_ptr(), q.data_ptr(), v.data_ptr(), out.data_ptr(), nullptr,
                                nullptr, graph->num_nodes, graph->num_edges, heads, d, dt, ws.data_ptr(),
                                (size_t)ws.numel(), current_stream(out)),
           "ga_dot_attention_sum");
  return out;
}

// edge_softmax_sum(SegmentMMEdgeDot(k, att, 0, q, 1, scale) / divisor,
//                  SegmentMMEdgeGather(v, msg, 0)): the message and reduce stages of an HGT
// layer (examples/HGT/HGT.py:35-53).  Both relation products are linear in a matrix per
// relation, so with at least two edges per (destination, relation) pair they are applied
// per pair instead of per edge:
//   score = <k[src], q[dst] (s A)^T>,  out[v] = sum_pairs (sum_{e in pair} a_e v[src]) M
// with one pass over the slots for scores, softmax inside the pair and weighted sum
// (ga_dot_attention_sum), the pairs of a destination weighed by the softmax of their
// log-sum-exps.  Graphs without such pairs and shapes outside those kernels run the
// three per-edge operators.
torch::Tensor relation_pair_attention(torch::Tensor k, torch::Tensor q, torch::Tensor v,
                                      torch::Tensor relation_att, torch::Tensor relation_msg,
                                      at::optional<torch::Tensor> scale, double divisor,
                                      const GraphPtr &graph) {
  auto per_edge = [&]() {
    torch::Tensor score = SegmentMMEdgeDot(k, relation_att, 0, q, 1, scale, graph);
    if (divisor != 1.0) score = score / divisor;
    return edge_softmax_sum(score, SegmentMMEdgeGather(v, relation_msg, 0, at::nullopt, graph),
                            graph);
  };
  // (T, D, D) matrices are one head
  const int64_t wd = relation_att.dim();
  const bool shapes = (wd == 3 || wd == 4) && relation_att.sizes() == relation_msg.sizes() &&
                      relation_att.size(wd - 2) == relation_att.size(wd - 1) && k.dim() == 2 &&
                      k.sizes() == q.sizes() && k.sizes() == v.sizes() && k.is_cuda() &&
                      q.is_cuda() && v.is_cuda() && relation_att.is_cuda() &&
                      relation_msg.is_cuda() && k.is_contiguous() && q.is_contiguous() &&
                      v.is_contiguous() && relation_msg.is_contiguous() &&
                      (k.scalar_type() == at::kFloat || k.scalar_type() == at::kBFloat16) &&
                      q.scalar_type() == k.scalar_type() && v.scalar_type() == k.scalar_type() &&
                      relation_att.scalar_type() == k.scalar_type() &&
                      relation_msg.scalar_type() == k.scalar_type() &&
                      relation_att.size(0) == graph->num_etypes &&
                      k.size(0) == graph->num_nodes &&
                      k.size(1) == (wd == 4 ? relation_att.size(1) : 1) * relation_att.size(wd - 1) &&
                      graph->etype_pointer.has_value();
  if (!shapes) return per_edge();
  const int64_t heads = wd == 4 ? relation_att.size(1) : 1, d = relation_att.size(wd - 1);
  const int64_t hid = heads * d;
  if (scale.has_value() && scale.value().numel() != graph->num_etypes * heads) return per_edge();
  const DGLGraph::RelationPairs &pairs = graph->relation_pairs();
  const int64_t n = graph->num_nodes, e = graph->num_edges, P = pairs.num_pairs;
  if (!pairs.valid || e < 2 * P) return per_edge();
  const int dt = feat_dtype(k, "k");
  const auto stream = current_stream(k);
  if (!relation_att.is_contiguous()) return per_edge();
  // the matrices as the query side needs them: transposed, times scale / divisor
  torch::Tensor att_t = torch::empty_like(relation_att);
  torch::Tensor sc;
  if (scale.has_value()) sc = scale.value().to(at::kFloat).contiguous();
  check_ga(ga_transpose_scale_blocks(relation_att.data_ptr(),
                                     sc.defined() ? sc.data_ptr<float>() : nullptr,
                                     (float)(1.0 / divisor), att_t.data_ptr(),
                                     graph->num_etypes * heads, d, dt, stream),
           "ga_transpose_scale_blocks");
  auto typed_rows = [&](const torch::Tensor &x, const torch::Tensor &index,
                        const torch::Tensor &w, torch::Tensor &y) {
    return ga_segment_mm_gather(pairs.type_pointer.data_ptr<int>(), graph->num_etypes,
                                x.data_ptr(), index.data_ptr<int64_t>(), w.data_ptr(),
                                y.data_ptr(), nullptr, nullptr, nullptr, nullptr, nullptr, P, heads,
                                d, d, dt, stream);
  };
  torch::Tensor q_pair = torch::empty({P, hid}, k.options());
  int rc = typed_rows(q, pairs.dst_by_type, att_t, q_pair);
  if (rc == GA_EUNSUPPORTED) return per_edge();
  check_ga(rc, "ga_segment_mm_gather");
  torch::Tensor ws = graph->workspace(std::max(
      {ga_gat_workspace_bytes(e, hid, heads), ga_softmax_workspace_bytes(P, heads),
       ga_spmm_workspace_bytes(P, hid)}));
  torch::Tensor v_pair = torch::empty({P, hid}, k.options());
  torch::Tensor lse = torch::empty({P, heads}, k.options().dtype(at::kFloat));
  rc = ga_dot_attention_sum(pairs.pair_pointer.data_ptr<int>(), pairs.pair_of_slot.data_ptr<int>(),
                            graph->in_node_indices.data_ptr<int>(),
                            pairs.rank_of_slot.data_ptr<int>(), k.data_ptr(), q_pair.data_ptr(),
                            v.data_ptr(), v_pair.data_ptr(), lse.data_ptr<float>(),
                            pairs.rank.data_ptr<int>(), P, e, heads, d, dt, ws.data_ptr(),
                            (size_t)ws.numel(), stream);
  if (rc == GA_EUNSUPPORTED) return per_edge();
  check_ga(rc, "ga_dot_attention_sum");
  // (the log-sum-exps were written in by_type order, the row order of m_pair)
  torch::Tensor m_pair = torch::empty({P, hid}, k.options());
  check_ga(typed_rows(v_pair, pairs.by_type, relation_msg, m_pair), "ga_segment_mm_gather");
  torch::Tensor out = torch::empty({n, hid}, k.options());
  check_ga(ga_edge_softmax_sum(pairs.dst_pointer.data_ptr<int>(), pairs.pair_dst.data_ptr<int>(),
                               pairs.rank.data_ptr<int>(), lse.data_ptr<float>(), m_pair.data_ptr(),
                               out.data_ptr(), n, P, heads, d, dt, ws.data_ptr(), (size_t)ws.numel(),
                               stream),
           "ga_edge_softmax_sum");
  return out;
}

// z = x @ w with the GAT attention terms from the same kernel (GAT.py:25-29);
// fp32 or bf16 storage, el / er always fp32.  Returns the C-ABI code so that a
// caller can fall back on GA_EUNSUPPORTED.
int project_attn(const torch::Tensor &x, const torch::Tensor &w, const torch::Tensor &a_l,
                 const torch::Tensor &a_r, int64_t heads, torch::Tensor &z, torch::Tensor &el,
                 torch::Tensor &er) {
  const int64_t rows = x.size(0), K = x.size(1), M = w.size(1);
  z = torch::empty({rows, M}, x.options());
  el = torch::empty({rows, heads}, x.options().dtype(at::kFloat));
  er = torch::empty({rows, heads}, x.options().dtype(at::kFloat));
  return ga_project_attn(x.data_ptr(), w.data_ptr(), a_l.data_ptr<float>(),
                         a_r.data_ptr<float>(), z.data_ptr(), el.data_ptr<float>(),
                         er.data_ptr<float>(), rows, K, M, heads,
                         x.scalar_type() == at::kFloat ? GA_F32 : GA_BF16, current_stream(x));
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> linear_attn(
    torch::Tensor x, torch::Tensor w, torch::Tensor a_l, torch::Tensor a_r) {
  check_input(x, "x");
  check_input(w, "weight");
  check_input(a_l, "a_l");
  check_input(a_r, "a_r");
  feat_dtype(x, "x");
  TORCH_CHECK(w.scalar_type() == x.scalar_type(), "x and weight must share a dtype");
  TORCH_CHECK(a_l.scalar_type() == at::kFloat && a_r.scalar_type() == at::kFloat,
              "a_l and a_r must be float32");
  TORCH_CHECK(x.dim() == 2 && w.dim() == 2 && w.size(0) == x.size(1), "weight must be (K, M)");
  const int64_t M = w.size(1);
  TORCH_CHECK(a_l.dim() == 2 && a_l.numel() == M && a_r.numel() == M && a_r.dim() == 2 &&
                  a_r.size(0) == a_l.size(0),
              "a_l and a_r must be (heads, M / heads)");
  torch::Tensor z, el, er;
  check_ga(project_attn(x, w, a_l, a_r, a_l.size(0), z, el, er), "ga_project_attn");
  return std::make_tuple(z, el, er);
}

// The dense head of a GAT layer after the split / reorder passes
// (GAT.py:25-29): z = h @ fc, el = z @ w_src, er = z @ w_dst with w_src / w_dst
// the two (M, 1) halves of the attention vector.  One kernel when the shape
// allows (fp32 or bf16, a single attention column, a width the kernels take);
// otherwise three GPU GEMMs through ATen, still on the device.  el / er are fp32
// either way (the aggregation that follows reads them as fp32).
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> gat_project(
    torch::Tensor h, torch::Tensor fc, torch::Tensor w_src, torch::Tensor w_dst) {
  check_input(h, "h");
  check_input(fc, "fc_weight");
  TORCH_CHECK(w_src.is_cuda() && w_dst.is_cuda(), "attention weights must be a CUDA tensor");
  TORCH_CHECK(h.dim() == 2 && fc.dim() == 2 && fc.size(0) == h.size(1), "fc_weight must be (K, M)");
  const int64_t M = fc.size(1);
  const bool candidate =
      (h.scalar_type() == at::kFloat || h.scalar_type() == at::kBFloat16) &&
      fc.scalar_type() == h.scalar_type() && w_src.dim() == 2 && w_dst.dim() == 2 &&
      w_src.size(1) == 1 && w_dst.size(1) == 1 && w_src.size(0) == M && w_dst.size(0) == M;
  if (candidate) {   // an (M, 1) column read as one (1, M) head vector
    torch::Tensor z, el, er;
    const int rc = project_attn(h, fc, w_src.to(at::kFloat).contiguous().view({1, M}),
                                w_dst.to(at::kFloat).contiguous().view({1, M}), 1, z, el, er);
    if (rc != GA_EUNSUPPORTED) {
      check_ga(rc, "ga_project_attn");
      return std::make_tuple(z, el, er);
    }
  }
  torch::Tensor z = at::mm(h, fc);
  return std::make_tuple(z, at::mm(z, w_src).to(at::kFloat), at::mm(z, w_dst).to(at::kFloat));
}

// Multi-head form of the same head: zv = (h @ fc).view(-1, heads, dim),
// el = sum(zv * a_l, 2, keepdim), er likewise, with a_l / a_r of heads * dim
// elements (any leading unit dimensions).  Returns zv (N, heads, dim) and
// el / er (N, heads, 1) fp32.
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> gat_project_heads(
    torch::Tensor h, torch::Tensor fc, torch::Tensor a_l, torch::Tensor a_r, int64_t heads,
    int64_t dim) {
  check_input(h, "h");
  check_input(fc, "fc_weight");
  TORCH_CHECK(a_l.is_cuda() && a_r.is_cuda(), "attention vectors must be a CUDA tensor");
  TORCH_CHECK(h.dim() == 2 && fc.dim() == 2 && fc.size(0) == h.size(1), "fc_weight must be (K, M)");
  TORCH_CHECK(heads > 0 && dim > 0 && fc.size(1) == heads * dim,
              "fc_weight must have heads * dim columns");
  TORCH_CHECK(a_l.numel() == heads * dim && a_r.numel() == heads * dim,
              "attention vectors must have heads * dim elements");
  const int64_t rows = h.size(0);
  const bool candidate = (h.scalar_type() == at::kFloat || h.scalar_type() == at::kBFloat16) &&
                         fc.scalar_type() == h.scalar_type();
  if (candidate) {
    torch::Tensor z, el, er;
    const int rc = project_attn(h, fc, a_l.to(at::kFloat).contiguous().view({heads, dim}),
                                a_r.to(at::kFloat).contiguous().view({heads, dim}), heads, z, el, er);
    if (rc != GA_EUNSUPPORTED) {
      check_ga(rc, "ga_project_attn");
      return std::make_tuple(z.view({rows, heads, dim}), el.view({rows, heads, 1}),
                             er.view({rows, heads, 1}));
    }
  }
  torch::Tensor zv = at::mm(h, fc).view({rows, heads, dim});
  torch::Tensor l = (zv * a_l.view({1, heads, dim})).sum(2, true).to(at::kFloat);
  torch::Tensor r = (zv * a_r.view({1, heads, dim})).sum(2, true).to(at::kFloat);
  return std::make_tuple(zv, l, r);
}

}  // namespace

TORCH_LIBRARY(my_classes, m) {
  m.class_<DGLGraph>("DGLGraph")
      .def(torch::init<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
                       torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
                       at::optional<torch::Tensor>, at::optional<torch::Tensor>>())
      .def("SetNtypePointer", &DGLGraph::SetNtypePointer)
      .def("SetEtypePointer", &DGLGraph::SetEtypePointer)
      .def("SetNtypeCOO", &DGLGraph::SetNtypeCOO)
      .def("SetEtypeCOO", &DGLGraph::SetEtypeCOO);
}

#define GRAPH_T "__torch__.torch.classes.my_classes.DGLGraph"

static auto registry =
    torch::RegisterOperators(
        "my_ops::SpMMEdge(Tensor x, int[] dim, bool k, int? t, " GRAPH_T " g) -> Tensor y",
        &SpMMEdge)
        .op("my_ops::SpMMSrc(Tensor x, int[] dim, bool k, int? t, " GRAPH_T " g) -> Tensor y",
            &SpMMSrc)
        .op("my_ops::gspmm_src_mul_e_sum(Tensor x, Tensor y, int[] dim, bool k, int? t, "
            GRAPH_T " g) -> Tensor z",
            &src_mul_e_sum)
        .op("my_ops::gspmm_dst_mul_e_sum(Tensor x, Tensor y, int[] dim, bool k, int? t, "
            GRAPH_T " g) -> Tensor z",
            &dst_mul_e_sum)
        .op("my_ops::gsddmm_u_add_v_mul_alpha(Tensor x, Tensor y, int alpha, " GRAPH_T
            " g) -> Tensor z",
            &u_add_v_mul_alpha)
        .op("my_ops::SegmentSoftmax(Tensor x, int dim, int? t, " GRAPH_T " g) -> Tensor y",
            &SegmentSoftmaxForward)
        .op("my_ops::SegmentMMNode(Tensor x, Tensor y, " GRAPH_T " g) -> Tensor z",
            &SegmentMMNode)
        .op("my_ops::SegmentMMEdge(Tensor x, Tensor y, " GRAPH_T " g) -> Tensor z",
            &SegmentMMEdge)
        .op("my_ops::BroadcastSrcNode(Tensor x, " GRAPH_T " g) -> Tensor y", &BroadcastSrcNode)
        .op("my_ops::BroadcastDstNode(Tensor x, " GRAPH_T " g) -> Tensor y", &BroadcastDstNode)
        .op("my_ops::BroadcastNodeType(Tensor x, " GRAPH_T " g) -> Tensor y", &BroadcastNodeType)
        .op("my_ops::BroadcastSrcNodeType(Tensor x, " GRAPH_T " g) -> Tensor y",
            &BroadcastSrcNodeType)
        .op("my_ops::BroadcastDstNodeType(Tensor x, " GRAPH_T " g) -> Tensor y",
            &BroadcastDstNodeType)
        .op("my_ops::BroadcastEdgeType(Tensor x, " GRAPH_T " g) -> Tensor y", &BroadcastEdgeType)
        .op("my_ops::get_feat_dim", &get_feat_dim)
        // additions of this build (no counterpart registered by the reference)
        .op("my_ops::gsddmm_u_dot_v(Tensor x, Tensor y, " GRAPH_T " g) -> Tensor z", &u_dot_v)
        .op("my_ops::gspmm(Tensor x, Tensor? y, str op, str reduce, " GRAPH_T " g) -> Tensor z",
            &gspmm)
        .op("my_ops::gspmm_bcast(Tensor? u, Tensor? e, str op, str reduce, bool reverse, " GRAPH_T
            " g) -> Tensor z",
            &gspmm_bcast)
        .op("my_ops::gsddmm(Tensor lhs, Tensor rhs, str op, str lhs_target, str rhs_target, "
            GRAPH_T " g) -> Tensor z",
            &gsddmm)
        .op("my_ops::gspmm_e_mul_e_sum(Tensor x, Tensor y, " GRAPH_T " g) -> Tensor z",
            &e_mul_e_sum)
        .op("my_ops::SpMMScaled(Tensor x, Tensor? row_scale, int activation, bool edge_rows, "
            GRAPH_T " g) -> Tensor y",
            &SpMMScaled)
        .op("my_ops::edge_softmax_sum(Tensor x, Tensor m, " GRAPH_T " g) -> Tensor z",
            &edge_softmax_sum)
        .op("my_ops::SegmentMMEdgeGather(Tensor x, Tensor w, int endpoint, Tensor? row_scale, "
            GRAPH_T " g) -> Tensor z",
            &SegmentMMEdgeGather)
        .op("my_ops::TypedSpMMEdge(Tensor x, Tensor w, Tensor? row_scale, " GRAPH_T
            " g) -> Tensor z",
            &TypedSpMMEdge)
        .op("my_ops::SegmentMMNodeStacked(Tensor x, Tensor[] ws, " GRAPH_T " g) -> Tensor[] zs",
            &SegmentMMNodeStacked)
        .op("my_ops::SegmentMMNodeScaled(Tensor x, Tensor w, Tensor row_scale, " GRAPH_T
            " g) -> Tensor z",
            &SegmentMMNodeScaled)
        .op("my_ops::SegmentMMNodeGated(Tensor x, Tensor w, Tensor gate, bool sigmoid, " GRAPH_T
            " g) -> Tensor z",
            &SegmentMMNodeGated)
        .op("my_ops::SegmentMMEdgeDot(Tensor x, Tensor w, int endpoint, Tensor q, "
            "int q_endpoint, Tensor? scale, " GRAPH_T " g) -> Tensor z",
            &SegmentMMEdgeDot)
        .op("my_ops::dot_attention_sum(Tensor k, Tensor q, Tensor v, " GRAPH_T " g) -> Tensor y",
            &dot_attention_sum)
        .op("my_ops::relation_pair_attention(Tensor k, Tensor q, Tensor v, Tensor att, Tensor msg, "
            "Tensor? scale, float divisor, " GRAPH_T " g) -> Tensor t",
            &relation_pair_attention)
        .op("my_ops::gat_aggregate(Tensor el, Tensor er, Tensor z, float slope, " GRAPH_T
            " g) -> Tensor y",
            &gat_aggregate)
        .op("my_ops::gat_aggregate_al(Tensor a_l, Tensor el, Tensor er, Tensor z, float slope, "
            GRAPH_T " g) -> Tensor y",
            &gat_aggregate_al)
        .op("my_ops::linear_attn(Tensor x, Tensor w, Tensor a_l, Tensor a_r) -> "
            "(Tensor z, Tensor el, Tensor er)",
            &linear_attn)
        .op("my_ops::gat_project(Tensor h, Tensor fc, Tensor w_src, Tensor w_dst) -> "
            "(Tensor z, Tensor el, Tensor er)",
            &gat_project)
        .op("my_ops::gat_project_heads(Tensor h, Tensor fc, Tensor a_l, Tensor a_r, int heads, "
            "int dim) -> (Tensor z, Tensor el, Tensor er)",
            &gat_project_heads);
