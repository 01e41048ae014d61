#include "execution_plan.hpp"

#include <algorithm>
#include <cstdlib>
#include <set>

namespace tracea_amd {

namespace {

using Id = uint64_t;

bool field(const Json &body, const char *key, long long *out) {
  const Json *f = body.find(key);
  if (f == nullptr || f->type != Json::Number) return false;
  *out = (long long)f->num;
  return true;
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }
int elem_bytes(int dt) { return dt == TRACEA_DTYPE_FLOAT32 ? 4 : 2; }

// First-fit arena with coalescing free list.
struct Arena {
  std::map<size_t, size_t> free_;  // offset -> size
  size_t top = 0;
  size_t take(size_t bytes) {
    size_t best = (size_t)-1, best_size = (size_t)-1;
    for (const auto &f : free_)
      if (f.second >= bytes && f.second < best_size) {
        best = f.first;
        best_size = f.second;
      }
    if (best != (size_t)-1) {
      free_.erase(best);
      if (best_size > bytes) free_[best + bytes] = best_size - bytes;
      return best;
    }
    // grow: a free block that ends at the top is extended instead of skipped
    if (!free_.empty()) {
      auto last = std::prev(free_.end());
      if (last->first + last->second == top) {
        const size_t off = last->first;
        free_.erase(last);
        top = off + bytes;
        return off;
      }
    }
    const size_t off = top;
    top += bytes;
    return off;
  }
  void give(size_t off, size_t bytes) {
    auto it = free_.emplace(off, bytes).first;
    auto next = std::next(it);
    if (next != free_.end() && it->first + it->second == next->first) {
      it->second += next->second;
      free_.erase(next);
    }
    if (it != free_.begin()) {
      auto prev = std::prev(it);
      if (prev->first + prev->second == it->first) {
        prev->second += it->second;
        free_.erase(it);
      }
    }
  }
};

}  // namespace

bool ExecutionPlan::compile(const Json &graph, int dtype, std::string *err) {
  steps_.clear();
  tensors_.clear();
  arena_size_ = 0;
  dtype_ = dtype;
  if (dtype != TRACEA_DTYPE_FLOAT16 && dtype != TRACEA_DTYPE_BFLOAT16) {
    *err = "plan dtype must be f16 or bf16";
    return false;
  }
  const Json *ops_j = graph.find("operators");
  const Json *deps_j = graph.find("dependencies");
  if (graph.type != Json::Object || !ops_j || ops_j->type != Json::Array || !deps_j || deps_j->type != Json::Array) {
    *err = "graph needs 'operators' and 'dependencies' arrays";
    return false;
  }
  std::map<Id, std::vector<Id>> producers, consumers;
  for (const Json &d : deps_j->arr) {
    if (d.type != Json::Array || d.arr.size() != 2 || d.arr[0].type != Json::Number || d.arr[1].type != Json::Number) {
      *err = "dependency must be [producer, consumer]";
      return false;
    }
    producers[(Id)d.arr[1].num].push_back((Id)d.arr[0].num);
    consumers[(Id)d.arr[0].num].push_back((Id)d.arr[1].num);
  }

  // ---- nodes ----
  std::map<Id, PlanStep> nodes;
  for (const Json &j : ops_j->arr) {
    if (j.type != Json::Object || j.obj.size() != 1 || j.obj[0].second.type != Json::Object) {
      *err = "operator must be an object with one variant key";
      return false;
    }
    PlanStep st;
    st.kind = j.obj[0].first;
    const Json &body = j.obj[0].second;
    long long id;
    if (!field(body, "op_id", &id)) {
      *err = "operator '" + st.kind + "' lacks op_id";
      return false;
    }
    st.id = (Id)id;
    if (const Json *nm = body.find("name")) st.name = nm->str;
    if (tensors_.count(st.id)) {
      *err = "duplicate op_id " + std::to_string(st.id);
      return false;
    }
    PlanTensor t;
    t.id = st.id;
    t.dtype = dtype;
    auto need = [&](std::initializer_list<const char *> keys) {
      int i = 0;
      for (const char *k : keys)
        if (!field(body, k, &st.g[i++])) {
          *err = st.kind + " '" + st.name + "' lacks field " + k;
          return false;
        }
      return true;
    };
    if (st.kind == "Input") {
      t.external = true;
      t.dtype = -1;  // whatever the caller binds
    } else if (st.kind == "Conv2d") {
      // g: n c h w k r s stride padding
      if (!need({"n", "c", "h", "w", "k", "r", "s", "stride", "padding"})) return false;
      if (st.g[7] <= 0) { *err = "Conv2d '" + st.name + "': stride must be positive"; return false; }
      const long long ho = (st.g[2] + 2 * st.g[8] - st.g[5]) / st.g[7] + 1, wo = (st.g[3] + 2 * st.g[8] - st.g[6]) / st.g[7] + 1;
      if (ho <= 0 || wo <= 0) { *err = "Conv2d '" + st.name + "' has an empty output"; return false; }
      st.g[9] = ho * wo;  // kept for describe()
      t.elems = st.g[0] * ho * wo * st.g[4];
      t.channels = (int)st.g[4];
    } else if (st.kind == "Gemm" || st.kind == "Linear") {
      // g: m n k batch
      if (!need({"m", "n", "k", "batch"})) return false;
      t.elems = st.g[3] * st.g[0] * st.g[1];
      t.channels = (int)st.g[1];
    } else if (st.kind == "BatchNorm" || st.kind == "GlobalAveragePool") {
      // g: n c h w
      if (!need({"n", "c", "h", "w"})) return false;
      t.elems = st.kind == "BatchNorm" ? st.g[0] * st.g[1] * st.g[2] * st.g[3] : st.g[0] * st.g[1];
      t.channels = (int)st.g[1];
      if (const Json *e = body.find("epsilon")) st.epsilon = (float)e->num;
    } else if (st.kind == "Relu" || st.kind == "Elementwise") {
      if (!need({"n"})) return false;
      t.elems = st.g[0];
      if (st.kind == "Elementwise") {
        const Json *k = body.find("kind");
        if (k == nullptr || k->str != "Add") {
          *err = "Elementwise '" + st.name + "': only kind \"Add\" has a kernel";
          return false;
        }
      }
    } else if (st.kind == "Softmax") {
      // size and row length come from the producer
    } else if (st.kind == "Attention") {
      // g: b s h d
      if (!need({"b", "s", "h", "d"})) return false;
      t.elems = st.g[0] * st.g[1] * st.g[2] * st.g[3];
      t.channels = (int)st.g[3];
    } else {
      *err = "operator kind '" + st.kind + "' has no kernel here";
      return false;
    }
    // epilogue list of a fused contraction
    if (const Json *ep = body.find("epilogue")) {
      if (ep->type != Json::Array) { *err = "epilogue must be an array"; return false; }
      for (const Json &e : ep->arr) {
        PlanEpilogue pe;
        if (e.type == Json::String) {
          if (e.str == "ReLU") pe.kind = TRACEA_EPI_OP_RELU;
          else if (e.str == "Gelu") pe.kind = TRACEA_EPI_OP_GELU;
          else if (e.str == "SiLU") pe.kind = TRACEA_EPI_OP_SILU;
          else if (e.str == "None") continue;
          else { *err = "epilogue entry \"" + e.str + "\" cannot be executed"; return false; }
        } else if (e.type == Json::Object && e.obj.size() == 1 && e.obj[0].first == "BatchNorm") {
          const Json &b = e.obj[0].second;
          long long ids[4];
          if (!field(b, "gamma_id", &ids[0]) || !field(b, "beta_id", &ids[1]) || !field(b, "mean_id", &ids[2]) ||
              !field(b, "var_id", &ids[3])) { *err = "BatchNorm epilogue lacks parameter ids"; return false; }
          pe.kind = TRACEA_EPI_OP_BATCHNORM;
          for (int i = 0; i < 4; ++i) pe.ids[i] = (Id)ids[i];
          pe.n_ids = 4;
          if (const Json *eps = b.find("epsilon")) pe.epsilon = (float)eps->num;
        } else if (e.type == Json::Object && e.obj.size() == 1 && e.obj[0].first == "ResidualAdd") {
          long long rid;
          if (!field(e.obj[0].second, "residual_ptr", &rid)) { *err = "ResidualAdd lacks residual_ptr"; return false; }
          pe.kind = TRACEA_EPI_OP_RESIDUAL_ADD;
          pe.ids[0] = (Id)rid;
          pe.n_ids = 1;
        } else {
          *err = "epilogue entry " + e.dump() + " cannot be executed";
          return false;
        }
        st.epilogue.push_back(pe);
      }
      if (st.epilogue.size() > TRACEA_MAX_EPILOGUE_OPS) {
        *err = st.kind + " '" + st.name + "' carries more than " + std::to_string(TRACEA_MAX_EPILOGUE_OPS) + " epilogue operators";
        return false;
      }
    }
    tensors_[st.id] = t;
    nodes[st.id] = st;
  }
  for (const auto &p : producers) {
    if (!nodes.count(p.first)) { *err = "dependency names unknown consumer " + std::to_string(p.first); return false; }
    for (Id src : p.second)
      if (!nodes.count(src)) { *err = "dependency names unknown producer " + std::to_string(src); return false; }
  }

  // ---- order: by operator id, as the reference schedules; a graph whose ids do not
  // follow its edges is sorted topologically (smallest ready id first) ----
  std::vector<Id> order;
  {
    std::map<Id, int> waiting;
    std::set<Id> ready;
    for (const auto &n : nodes) {
      waiting[n.first] = (int)producers[n.first].size();
      if (waiting[n.first] == 0) ready.insert(n.first);
    }
    while (!ready.empty()) {
      const Id id = *ready.begin();
      ready.erase(ready.begin());
      order.push_back(id);
      for (Id c : consumers[id])
        if (--waiting[c] == 0) ready.insert(c);
    }
    if (order.size() != nodes.size()) { *err = "graph has a cycle"; return false; }
  }

  // ---- data inputs, sizes that come from producers ----
  for (Id id : order) {
    PlanStep &st = nodes[id];
    if (st.kind == "Input") continue;
    std::set<Id> side;
    for (const PlanEpilogue &pe : st.epilogue)
      for (int i = 0; i < pe.n_ids; ++i) {
        side.insert(pe.ids[i]);
        if (!tensors_.count(pe.ids[i])) { *err = st.kind + " '" + st.name + "': epilogue names unknown tensor " + std::to_string(pe.ids[i]); return false; }
      }
    for (Id p : producers[id])
      if (!side.count(p)) st.inputs.push_back(p);
    PlanTensor &out = tensors_[id];
    const size_t want = st.kind == "Elementwise" ? 2 : st.kind == "Attention" ? 3 : st.kind == "BatchNorm" ? 5 : 1;
    if (st.inputs.size() != want) {
      *err = st.kind + " '" + st.name + "' needs " + std::to_string(want) + " inputs, the graph gives " + std::to_string(st.inputs.size());
      return false;
    }
    const PlanTensor &in0 = tensors_[st.inputs[0]];
    if (st.kind == "Relu" || st.kind == "Elementwise") {
      out.channels = in0.channels > 0 && out.elems % in0.channels == 0 ? in0.channels : (out.elems % 8 == 0 ? 8 : 1);
    } else if (st.kind == "Softmax") {
      if (in0.elems <= 0 || in0.channels <= 0) { *err = "Softmax '" + st.name + "': the size of its input is not known"; return false; }
      out.elems = in0.elems;
      out.channels = in0.channels;
    }
    if (st.kind == "Conv2d" && st.g[1] % 8 != 0) {
      *err = "Conv2d '" + st.name + "': input channels must be a multiple of 8 (pad the tensor and the filters with zero channels)";
      return false;
    }
    // a known producer size must agree with what this node reads
    long long reads = 0;
    if (st.kind == "Conv2d") reads = st.g[0] * st.g[2] * st.g[3] * st.g[1];
    else if (st.kind == "Gemm" || st.kind == "Linear") reads = st.g[3] * st.g[0] * st.g[2];
    else if (st.kind == "GlobalAveragePool") reads = st.g[0] * st.g[1] * st.g[2] * st.g[3];
    else reads = out.elems;  // element-wise nodes, Attention, Softmax (sized from its producer above)
    if (!in0.external && in0.elems != reads) {
      *err = st.kind + " '" + st.name + "' reads " + std::to_string(reads) + " elements, its producer writes " + std::to_string(in0.elems);
      return false;
    }
    // what this node reads from Input nodes, for bind_sized: data in the plan's type, BatchNorm
    // parameters as float32 channel vectors (gamma, beta, mean, var, in that order: the order of a
    // BatchNorm node's dependency list after its data input, and of the ids of a fused BatchNorm)
    auto needs = [&](Id id, long long elems, int dt) {
      PlanTensor &p = tensors_[id];
      if (!p.external || elems <= 0) return;
      const long long bytes = elems * (long long)elem_bytes(dt);
      if (bytes > p.need_bytes) p.need_bytes = bytes;
      p.need_dtype = dt;
    };
    needs(st.inputs[0], reads, dtype_);
    if (st.kind == "Elementwise") needs(st.inputs[1], out.elems, dtype_);
    if (st.kind == "Attention") { needs(st.inputs[1], out.elems, dtype_); needs(st.inputs[2], out.elems, dtype_); }
    if (st.kind == "BatchNorm")
      for (int i = 1; i < 5; ++i) needs(st.inputs[i], out.channels, TRACEA_DTYPE_FLOAT32);
    for (const PlanEpilogue &pe : st.epilogue) {
      if (pe.kind == TRACEA_EPI_OP_BATCHNORM)
        for (int i = 0; i < pe.n_ids; ++i) needs(pe.ids[i], out.channels, TRACEA_DTYPE_FLOAT32);
      if (pe.kind == TRACEA_EPI_OP_RESIDUAL_ADD) needs(pe.ids[0], out.elems, dtype_);
    }
  }

  // ---- steps, liveness, arena ----
  std::map<Id, int> step_of;
  for (Id id : order)
    if (nodes[id].kind != "Input") {
      step_of[id] = (int)steps_.size();
      steps_.push_back(nodes[id]);
    }
  // ---- a classifier head in one launch: a GlobalAveragePool node read by one Linear node only (batch 1 of the
  // Linear's geometry, the pooled channels as its K) is taken over by that Linear step, which computes the
  // means itself and still writes them to the pooling node's place.  TRACEA_PLAN_SPLIT_HEAD=1 at compile
  // keeps the two launches. ----
  {
    const char *keep = getenv("TRACEA_PLAN_SPLIT_HEAD");
    for (size_t i = 0; i + 1 < steps_.size() && !(keep && keep[0] == '1'); ++i) {
      PlanStep &pool = steps_[i], &lin = steps_[i + 1];
      if (pool.kind != "GlobalAveragePool" || lin.kind != "Linear" || lin.inputs.size() != 1 || lin.inputs[0] != pool.id) continue;
      if (consumers[pool.id].size() != 1 || lin.g[3] * lin.g[0] != pool.g[0] || lin.g[2] != pool.g[1] || pool.g[1] > 8192) continue;
      bool side = false;  // (the means must not be an operand of the Linear's own chain)
      for (const PlanEpilogue &pe : lin.epilogue)
        for (int k = 0; k < pe.n_ids; ++k) side = side || pe.ids[k] == pool.id;
      if (side) continue;
      lin.pool_id = pool.id;
      lin.pool_hw = pool.g[2] * pool.g[3];
      lin.inputs[0] = pool.inputs[0];
      steps_.erase(steps_.begin() + (long)i);
    }
  }
  const int n_steps = (int)steps_.size();
  // ---- neighbours that may run side by side: two contractions of which the second reads nothing the first
  // writes (a block's first convolution and its shortcut convolution).  Off unless TRACEA_PLAN_SIDE_BY_SIDE=1
  // is set when the plan is compiled: measured on ResNet-18 replayed as a HIP graph on one MI355X, the three
  // forks and joins cost more than the overlap gains (batch 1: 235 us against 215 serial; batch 32: 300
  // against 295) ----
  {
    auto heavy = [](const PlanStep &s) { return s.kind == "Conv2d" || s.kind == "Gemm" || s.kind == "Linear"; };
    auto reads = [](const PlanStep &s, Id t) {
      for (Id i : s.inputs)
        if (i == t) return true;
      for (const PlanEpilogue &pe : s.epilogue)
        for (int k = 0; k < pe.n_ids; ++k)
          if (pe.ids[k] == t) return true;
      return false;
    };
    const char *pairs = getenv("TRACEA_PLAN_SIDE_BY_SIDE");
    for (int i = 0; i + 1 < n_steps && pairs && pairs[0] == '1'; ++i)
      if (steps_[i].fork == 0 && heavy(steps_[i]) && heavy(steps_[i + 1]) && !reads(steps_[i + 1], steps_[i].id)) {
        steps_[i].fork = 1;
        steps_[i + 1].fork = 2;
        ++i;
      }
  }
  for (int i = 0; i < n_steps; ++i) {
    tensors_[steps_[i].id].born = i;
    if (steps_[i].pool_id != 0) {
      tensors_[steps_[i].pool_id].born = i;
      tensors_[steps_[i].pool_id].last_use = i;
    }
    auto touch = [&](Id t) {
      PlanTensor &pt = tensors_[t];
      if (!pt.external && pt.last_use < i) pt.last_use = i;
    };
    for (Id t : steps_[i].inputs) touch(t);
    for (const PlanEpilogue &pe : steps_[i].epilogue)
      for (int k = 0; k < pe.n_ids; ++k) touch(pe.ids[k]);
  }
  // what the first step of a side-by-side pair reads last stays until the second is done too (the second's
  // output must not land on memory the first still reads)
  for (int i = 0; i + 1 < n_steps; ++i)
    if (steps_[i].fork == 1)
      for (auto &t : tensors_)
        if (!t.second.external && t.second.last_use == i) t.second.last_use = i + 1;
  Arena arena;
  for (int i = 0; i < n_steps; ++i) {
    PlanTensor &out = tensors_[steps_[i].id];
    if (out.last_use < 0) out.last_use = n_steps;  // nobody reads it: a result of the graph
    out.bytes = align256((size_t)out.elems * elem_bytes(out.dtype));
    out.offset = arena.take(out.bytes);
    if (steps_[i].pool_id != 0) {
      PlanTensor &pt = tensors_[steps_[i].pool_id];
      pt.bytes = align256((size_t)pt.elems * elem_bytes(pt.dtype));
      pt.offset = arena.take(pt.bytes);
    }
    for (auto &t : tensors_) {
      PlanTensor &pt = t.second;
      if (!pt.external && pt.born >= 0 && pt.born <= i && pt.last_use == i) arena.give(pt.offset, pt.bytes);
    }
  }
  arena_size_ = arena.top;
  int dev = -1;
  if (hipGetDevice(&dev) == hipSuccess) (void)ensure_side(dev, nullptr);  // best effort: run() tries again
  else (void)hipGetLastError();
  return true;
}

ExecutionPlan::~ExecutionPlan() {
  if (ev_fork_) (void)hipEventDestroy((hipEvent_t)ev_fork_);
  if (ev_join_) (void)hipEventDestroy((hipEvent_t)ev_join_);
  if (side_stream_) (void)hipStreamDestroy((hipStream_t)side_stream_);
}

// The side stream and its two events on `device` (current when this is called).  Nothing is created while
// `stream` is being captured: creation calls are not allowed then, and the run stays on one stream.
bool ExecutionPlan::ensure_side(int device, void *stream) const {
  if (side_stream_ != nullptr && side_device_ == device) return true;
  bool any = false;
  for (const PlanStep &st : steps_) any = any || st.fork != 0;
  if (!any) return false;
  if (stream != nullptr) {
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing((hipStream_t)stream, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone) {
      (void)hipGetLastError();
      return false;
    }
  }
  if (ev_fork_) (void)hipEventDestroy((hipEvent_t)ev_fork_);
  if (ev_join_) (void)hipEventDestroy((hipEvent_t)ev_join_);
  if (side_stream_) (void)hipStreamDestroy((hipStream_t)side_stream_);
  ev_fork_ = ev_join_ = side_stream_ = nullptr;
  side_device_ = -1;
  hipStream_t s = nullptr;
  hipEvent_t a = nullptr, b = nullptr;
  if (hipStreamCreateWithFlags(&s, hipStreamNonBlocking) != hipSuccess || hipEventCreateWithFlags(&a, hipEventDisableTiming) != hipSuccess ||
      hipEventCreateWithFlags(&b, hipEventDisableTiming) != hipSuccess) {
    (void)hipGetLastError();
    if (a) (void)hipEventDestroy(a);
    if (b) (void)hipEventDestroy(b);
    if (s) (void)hipStreamDestroy(s);
    return false;
  }
  side_stream_ = s; ev_fork_ = a; ev_join_ = b;
  side_device_ = device;
  return true;
}

Json ExecutionPlan::describe() const {
  Json root = Json::make_obj();
  root.set("arena_size", Json::make_num((double)arena_size_));
  Json steps = Json::make_arr();
  for (const PlanStep &st : steps_) {
    const PlanTensor &t = tensors_.at(st.id);
    Json s = Json::make_obj();
    s.set("op_id", Json::make_num((double)st.id));
    s.set("kind", Json::make_str(st.kind));
    s.set("name", Json::make_str(st.name));
    Json in = Json::make_arr();
    for (Id i : st.inputs) in.arr.push_back(Json::make_num((double)i));
    s.set("inputs", in);
    Json side = Json::make_arr();
    for (const PlanEpilogue &pe : st.epilogue) {
      Json e = Json::make_obj();
      e.set("kind", Json::make_num(pe.kind));
      Json ids = Json::make_arr();
      for (int k = 0; k < pe.n_ids; ++k) ids.arr.push_back(Json::make_num((double)pe.ids[k]));
      e.set("tensors", ids);
      side.arr.push_back(e);
    }
    s.set("epilogue", side);
    s.set("offset", Json::make_num((double)t.offset));
    s.set("bytes", Json::make_num((double)t.bytes));
    s.set("elements", Json::make_num((double)t.elems));
    s.set("last_use", Json::make_num(t.last_use));
    s.set("pooled_from", Json::make_num((double)st.pool_id));
    s.set("side_by_side", Json::make_str(st.fork == 1 ? "first" : st.fork == 2 ? "second" : "no"));
    steps.arr.push_back(s);
  }
  root.set("steps", steps);
  // plan.rs:17: LogicalID -> (offset, size in bytes)
  Json outs = Json::make_obj();
  for (const auto &t : tensors_)
    if (!t.second.external) {
      Json pair = Json::make_arr();
      pair.arr.push_back(Json::make_num((double)t.second.offset));
      pair.arr.push_back(Json::make_num((double)((size_t)t.second.elems * elem_bytes(t.second.dtype))));
      outs.set(std::to_string(t.first), pair);
    }
  root.set("output_map", outs);
  return root;
}

bool ExecutionPlan::output(uint64_t op_id, size_t *offset, size_t *bytes) const {
  auto it = tensors_.find(op_id);
  if (it == tensors_.end() || it->second.external) return false;
  *offset = it->second.offset;
  *bytes = (size_t)it->second.elems * elem_bytes(it->second.dtype);
  return true;
}

TraceaStatus ExecutionPlan::bind(uint64_t op_id, const std::string &slot, void *ptr) {
  if (ptr == nullptr) return fail(TRACEA_INVALID_PARAMS, "tracea_plan_bind: NULL pointer for op %llu", (unsigned long long)op_id);
  if (slot == "input") {
    auto it = tensors_.find(op_id);
    if (it == tensors_.end() || !it->second.external)
      return fail(TRACEA_INVALID_PARAMS, "tracea_plan_bind: op %llu is not an Input node", (unsigned long long)op_id);
    it->second.ext = ptr;
    return TRACEA_SUCCESS;
  }
  const int layout = slot == "weight" ? 0 : (slot == "weight_rsck" || slot == "weight_t") ? 1 : -1;
  if (layout < 0) return fail(TRACEA_INVALID_PARAMS, "tracea_plan_bind: unknown slot '%s'", slot.c_str());
  for (PlanStep &st : steps_)
    if (st.id == op_id) {
      if (st.kind != "Conv2d" && st.kind != "Gemm" && st.kind != "Linear")
        return fail(TRACEA_INVALID_PARAMS, "tracea_plan_bind: %s nodes take no weight", st.kind.c_str());
      st.weight = ptr;
      st.weight_layout = layout;
      return TRACEA_SUCCESS;
    }
  return fail(TRACEA_INVALID_PARAMS, "tracea_plan_bind: no step with op_id %llu", (unsigned long long)op_id);
}

TraceaStatus ExecutionPlan::bind_sized(uint64_t op_id, const std::string &slot, void *ptr, size_t bytes, int dtype) {
  if (slot == "input") {
    auto it = tensors_.find(op_id);
    if (it != tensors_.end() && it->second.external) {
      const PlanTensor &t = it->second;
      if (t.need_bytes > 0 && (long long)bytes < t.need_bytes)
        return fail(TRACEA_INVALID_PARAMS, "tracea_plan_bind: the tensor bound to input %llu holds %zu bytes, the plan reads %lld",
                    (unsigned long long)op_id, bytes, t.need_bytes);
      if (t.need_dtype >= 0 && dtype >= 0 && dtype != t.need_dtype)
        return fail(TRACEA_INVALID_PARAMS, "tracea_plan_bind: the tensor bound to input %llu has element type %d, the plan reads it as %d",
                    (unsigned long long)op_id, dtype, t.need_dtype);
    }
  } else {
    for (const PlanStep &st : steps_)
      if (st.id == op_id && (st.kind == "Conv2d" || st.kind == "Gemm" || st.kind == "Linear")) {
        const long long elems = st.kind == "Conv2d" ? st.g[4] * st.g[5] * st.g[6] * st.g[1] : st.g[2] * st.g[1];
        const long long need = elems * (long long)elem_bytes(dtype_);
        if ((long long)bytes < need)
          return fail(TRACEA_INVALID_PARAMS, "tracea_plan_bind: the weights bound to %s '%s' hold %zu bytes, the node reads %lld",
                      st.kind.c_str(), st.name.c_str(), bytes, need);
        if (dtype >= 0 && dtype != dtype_)
          return fail(TRACEA_INVALID_PARAMS, "tracea_plan_bind: the weights bound to %s '%s' have element type %d, the plan computes in %d",
                      st.kind.c_str(), st.name.c_str(), dtype, dtype_);
      }
  }
  return bind(op_id, slot, ptr);
}

void *ExecutionPlan::address(uint64_t id, void *arena) const {
  const PlanTensor &t = tensors_.at(id);
  return t.external ? t.ext : (void *)((char *)arena + t.offset);
}

TraceaStatus ExecutionPlan::run(void *arena, int device, void *stream) const {
  if (arena == nullptr && arena_size_ > 0) return fail(TRACEA_INVALID_PARAMS, "tracea_plan_run: arena is NULL");
  if ((((uintptr_t)arena) & 255) != 0) return fail(TRACEA_INVALID_PARAMS, "tracea_plan_run: arena must be 256-byte aligned");
  const TraceaDType dt = (TraceaDType)dtype_;
  // everything a step needs must be bound before the first launch
  for (const PlanStep &st : steps_) {
    for (Id i : st.inputs)
      if (tensors_.at(i).external && tensors_.at(i).ext == nullptr)
        return fail(TRACEA_INVALID_PARAMS, "tracea_plan_run: Input %llu (read by '%s') is not bound", (unsigned long long)i, st.name.c_str());
    for (const PlanEpilogue &pe : st.epilogue)
      for (int k = 0; k < pe.n_ids; ++k)
        if (tensors_.at(pe.ids[k]).external && tensors_.at(pe.ids[k]).ext == nullptr)
          return fail(TRACEA_INVALID_PARAMS, "tracea_plan_run: Input %llu (epilogue of '%s') is not bound", (unsigned long long)pe.ids[k], st.name.c_str());
    if ((st.kind == "Conv2d" || st.kind == "Gemm" || st.kind == "Linear") && st.weight == nullptr)
      return fail(TRACEA_INVALID_PARAMS, "tracea_plan_run: '%s' has no weight bound", st.name.c_str());
  }
  // the node kernels below launch on the current device; the caller's choice is put back
  struct DeviceGuard {
    int prev = -1;
    ~DeviceGuard() { if (prev >= 0) (void)hipSetDevice(prev); }
  } guard;
  {
    int cur = -1;
    if (hipGetDevice(&cur) == hipSuccess && cur != device) {
      hipError_t e = hipSetDevice(device);
      if (e != hipSuccess) return fail(TRACEA_CUDA_ERROR, "tracea_plan_run: %s", hipGetErrorString(e));
      guard.prev = cur;
    }
  }
  auto view = [&](void *ptr, int rank, const uint64_t *shape, const int64_t *stride, TraceaDType d) {
    TraceaTensorView v{};
    v.ptr = ptr; v.rank = (uint32_t)rank; v.shape = shape; v.stride = stride; v.dtype = d; v.device_id = device;
    return v;
  };
  const bool forking = ensure_side(device, stream);
  void *const main_stream = stream;
  for (const PlanStep &st : steps_) {
    // a pair of independent neighbours: the side stream picks up behind everything launched so far, runs the
    // second step, and the main stream waits for it before going on
    if (forking && st.fork == 1) {
      hipError_t e = hipEventRecord((hipEvent_t)ev_fork_, (hipStream_t)main_stream);
      if (e == hipSuccess) e = hipStreamWaitEvent((hipStream_t)side_stream_, (hipEvent_t)ev_fork_, 0);
      if (e != hipSuccess) return fail(TRACEA_CUDA_ERROR, "tracea_plan_run: fork in front of '%s': %s", st.name.c_str(), hipGetErrorString(e));
    }
    stream = forking && st.fork == 2 ? side_stream_ : main_stream;
    void *out = address(st.id, arena);
    const PlanTensor &ot = tensors_.at(st.id);
    TraceaEpilogueOp ops[TRACEA_MAX_EPILOGUE_OPS];
    uint32_t n_ops = 0;
    for (const PlanEpilogue &pe : st.epilogue) {
      TraceaEpilogueOp o{};
      o.kind = (TraceaEpilogueOpKind)pe.kind;
      o.dtype = TRACEA_DTYPE_FLOAT32;
      o.epsilon = pe.epsilon;
      const void *p[4] = {nullptr, nullptr, nullptr, nullptr};
      for (int k = 0; k < pe.n_ids; ++k) p[k] = address(pe.ids[k], arena);
      o.p0 = p[0]; o.p1 = p[1]; o.p2 = p[2]; o.p3 = p[3];
      if (pe.kind == TRACEA_EPI_OP_RESIDUAL_ADD) {
        const PlanTensor &rt = tensors_.at(pe.ids[0]);
        o.dtype = rt.external ? dt : (TraceaDType)rt.dtype;  // a skip input has the plan's dtype
        o.ld = 0;
      }
      ops[n_ops++] = o;
    }
    TraceaStatus status = TRACEA_SUCCESS;
    if (st.kind == "Conv2d") {
      const long long n = st.g[0], c = st.g[1], h = st.g[2], w = st.g[3], k = st.g[4], r = st.g[5], s = st.g[6];
      const long long ho = (h + 2 * st.g[8] - r) / st.g[7] + 1, wo = (w + 2 * st.g[8] - s) / st.g[7] + 1;
      const uint64_t xs[4] = {(uint64_t)n, (uint64_t)h, (uint64_t)w, (uint64_t)c};
      const uint64_t ws[4] = {(uint64_t)k, (uint64_t)r, (uint64_t)s, (uint64_t)c};
      const uint64_t os[4] = {(uint64_t)n, (uint64_t)ho, (uint64_t)wo, (uint64_t)k};
      const int64_t wst[4] = {1, s * c * k, c * k, k};  // [R,S,C,K] storage
      TraceaTensorView o = view(out, 4, os, nullptr, dt);
      TraceaConv2dParams p{};
      p.stride_h = p.stride_w = (uint32_t)st.g[7];
      p.padding_h = p.padding_w = (uint32_t)st.g[8];
      p.dilation_h = p.dilation_w = 1;
      p.groups = 1;
      p.stream = stream;
      status = dispatch_conv2d_ops(view(address(st.inputs[0], arena), 4, xs, nullptr, dt),
                                   view((void *)st.weight, 4, ws, st.weight_layout ? wst : nullptr, dt), &o, p, ops, n_ops);
    } else if (st.kind == "Linear" && st.pool_id != 0) {
      PoolLinearArgs a{};
      a.x = address(st.inputs[0], arena);
      a.w = st.weight;
      a.out = out;
      a.pooled = address(st.pool_id, arena);
      a.dtype = a.out_dtype = dt;
      a.batch = (int)(st.g[3] * st.g[0]); a.hw = (int)st.pool_hw; a.channels = (int)st.g[2]; a.n_out = (int)st.g[1];
      a.w_ld = st.weight_layout ? st.g[2] : st.g[1];  // [N,K] storage: k contiguous; else [K,N]
      EpilogueChain chain{};
      status = dispatch_lower_chain("tracea_plan_run", ops, n_ops, st.g[1], &chain);
      if (status == TRACEA_SUCCESS) {
        a.epi = chain;
        const int e = launch_pool_linear(a, st.weight_layout != 0, (hipStream_t)stream);
        if (e != 0) status = fail(TRACEA_CUDA_ERROR, "tracea_plan_run: '%s': %s", st.name.c_str(), hipGetErrorString((hipError_t)e));
      }
    } else if (st.kind == "Gemm" || st.kind == "Linear") {
      const long long m = st.g[3] * st.g[0], n = st.g[1], k = st.g[2];
      const uint64_t as[2] = {(uint64_t)m, (uint64_t)k}, bs[2] = {(uint64_t)k, (uint64_t)n}, cs[2] = {(uint64_t)m, (uint64_t)n};
      const int64_t bt[2] = {1, k};  // [N,K] storage
      TraceaTensorView c = view(out, 2, cs, nullptr, dt);
      TraceaGemmParams p{};
      p.stream = stream;
      status = dispatch_gemm_ops(view(address(st.inputs[0], arena), 2, as, nullptr, dt),
                                 view((void *)st.weight, 2, bs, st.weight_layout ? bt : nullptr, dt), &c, p, ops, n_ops);
    } else if (st.kind == "Attention") {
      const uint64_t sh[4] = {(uint64_t)st.g[0], (uint64_t)st.g[2], (uint64_t)st.g[1], (uint64_t)st.g[3]};  // [B,H,S,D]
      TraceaTensorView o = view(out, 4, sh, nullptr, dt);
      TraceaAttentionParams p{};
      p.stream = stream;
      status = dispatch_attention(view(address(st.inputs[0], arena), 4, sh, nullptr, dt),
                                  view(address(st.inputs[1], arena), 4, sh, nullptr, dt),
                                  view(address(st.inputs[2], arena), 4, sh, nullptr, dt), &o, p);
    } else {
      int e = 0;
      if (st.kind == "GlobalAveragePool") {
        e = launch_global_avg_pool(address(st.inputs[0], arena), out, dt, dt, (int)st.g[0], (int)(st.g[2] * st.g[3]),
                                   (int)st.g[1], (hipStream_t)stream);
      } else if (st.kind == "Softmax") {
        e = launch_softmax_rows(address(st.inputs[0], arena), out, dt, dt, ot.elems / ot.channels, ot.channels,
                                (hipStream_t)stream);
      } else {
        ChainApplyArgs a{};
        a.x = address(st.inputs[0], arena);
        a.out = out;
        a.x_dtype = a.out_dtype = dt;
        a.channels = ot.channels;
        a.rows = ot.elems / ot.channels;
        EpilogueOpDev d{};
        d.dtype = DT_F32;
        if (st.kind == "Relu") {
          d.kind = TRACEA_EPI_OP_RELU;
        } else if (st.kind == "Elementwise") {
          d.kind = TRACEA_EPI_OP_RESIDUAL_ADD;
          d.p0 = address(st.inputs[1], arena);
          d.dtype = dt;
          d.ld = ot.channels;
        } else {  // BatchNorm: x, gamma, beta, mean, var
          d.kind = TRACEA_EPI_OP_BATCHNORM;
          d.p0 = address(st.inputs[1], arena); d.p1 = address(st.inputs[2], arena);
          d.p2 = address(st.inputs[3], arena); d.p3 = address(st.inputs[4], arena);
          d.epsilon = st.epsilon;
        }
        a.epi.n_ops = 1;
        a.epi.ops[0] = d;
        e = launch_chain_apply(a, (hipStream_t)stream);
      }
      if (e != 0) status = fail(TRACEA_CUDA_ERROR, "tracea_plan_run: '%s': %s", st.name.c_str(), hipGetErrorString((hipError_t)e));
    }
    if (forking && st.fork == 2) {
      // (joined also after a failed launch: a capture must not end with the side stream still forked)
      hipError_t e = hipEventRecord((hipEvent_t)ev_join_, (hipStream_t)side_stream_);
      if (e == hipSuccess) e = hipStreamWaitEvent((hipStream_t)main_stream, (hipEvent_t)ev_join_, 0);
      if (e != hipSuccess && status == TRACEA_SUCCESS)
        status = fail(TRACEA_CUDA_ERROR, "tracea_plan_run: join behind '%s': %s", st.name.c_str(), hipGetErrorString(e));
    }
    if (status != TRACEA_SUCCESS) return status;
  }
  return TRACEA_SUCCESS;
}

}  // namespace tracea_amd
