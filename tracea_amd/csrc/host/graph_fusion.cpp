#include "graph_fusion.hpp"

#include <algorithm>
#include <map>
#include <set>
#include <vector>

namespace tracea_amd {

namespace {

using Id = uint64_t;
using Edges = std::map<Id, std::vector<Id>>;

struct Node {
  std::string kind;  // variant name: "Conv2d", "Relu", ...
  Json body;         // the variant's fields
  Id id = 0;
};

bool read_node(const Json &j, Node *out, std::string *err) {
  if (j.type != Json::Object || j.obj.size() != 1 || j.obj[0].second.type != Json::Object) {
    *err = "operator must be an object with one variant key";
    return false;
  }
  out->kind = j.obj[0].first;
  out->body = j.obj[0].second;
  const Json *id = out->body.find("op_id");
  if (id == nullptr || id->type != Json::Number) {
    *err = "operator '" + out->kind + "' lacks op_id";
    return false;
  }
  out->id = (Id)id->num;
  return true;
}

bool accepts_epilogue(const Node &n) { return n.kind == "Conv2d" || n.kind == "Linear" || n.kind == "Gemm"; }

// The epilogue entry `consumer` turns into when merged into `producer`, and the
// producer count the merge requires; false when the consumer cannot be merged.
bool map_to_epilogue(const Node &consumer, const Edges &reverse, Id producer, const std::map<Id, Id> &fused_into,
                     Json *entry, size_t *need_producers) {
  const auto it = reverse.find(consumer.id);
  if (consumer.kind == "Relu") {
    *entry = Json::make_str("ReLU");
    *need_producers = 1;
    return true;
  }
  if (consumer.kind == "BatchNorm") {
    if (it == reverse.end()) return false;
    const std::vector<Id> &p = it->second;  // x, gamma, beta, mean, var in dependency order
    auto at = [&](size_t i) { return Json::make_num(i < p.size() ? (double)p[i] : 0.0); };
    Json f = Json::make_obj();
    f.set("op_id", Json::make_num((double)consumer.id));
    f.set("gamma_id", at(1));
    f.set("beta_id", at(2));
    f.set("mean_id", at(3));
    f.set("var_id", at(4));
    const Json *eps = consumer.body.find("epsilon");
    f.set("epsilon", eps ? *eps : Json::make_num(1e-5));
    *entry = Json::make_obj();
    entry->set("BatchNorm", f);
    *need_producers = 5;
    return true;
  }
  if (consumer.kind == "Elementwise") {
    const Json *kind = consumer.body.find("kind");
    if (kind == nullptr || kind->str != "Add" || it == reverse.end()) return false;
    Id skip = 0;
    bool found = false;
    for (Id p : it->second)
      if (p != producer) {
        skip = p;
        found = true;
        break;
      }
    if (!found) return false;
    // a skip input that was itself merged away is represented by the node it went into
    for (auto f = fused_into.find(skip); f != fused_into.end(); f = fused_into.find(skip)) skip = f->second;
    Json fields = Json::make_obj();
    fields.set("residual_ptr", Json::make_num((double)skip));
    *entry = Json::make_obj();
    entry->set("ResidualAdd", fields);
    *need_producers = 2;
    return true;
  }
  return false;
}

}  // namespace

bool fuse_graph(Json *graph, std::string *err) {
  const Json *ops_j = graph->find("operators");
  const Json *deps_j = graph->find("dependencies");
  if (graph->type != Json::Object || !ops_j || ops_j->type != Json::Array || !deps_j ||
      deps_j->type != Json::Array) {
    *err = "graph needs 'operators' and 'dependencies' arrays";
    return false;
  }
  std::vector<Node> current;
  for (const Json &j : ops_j->arr) {
    Node n;
    if (!read_node(j, &n, err)) return false;
    current.push_back(n);
  }
  Edges adj, reverse;
  for (const Json &d : deps_j->arr) {
    if (d.type != Json::Array || d.arr.size() != 2 || d.arr[0].type != Json::Number ||
        d.arr[1].type != Json::Number) {
      *err = "dependency must be [producer, consumer]";
      return false;
    }
    const Id src = (Id)d.arr[0].num, dst = (Id)d.arr[1].num;
    adj[src].push_back(dst);
    reverse[dst].push_back(src);
  }

  std::set<Id> removed;
  std::map<Id, Id> fused_into;
  bool modified = true;
  while (modified) {
    modified = false;
    std::vector<Node> next;
    for (const Node &op : current) {
      if (removed.count(op.id)) continue;
      bool merged = false;
      if (accepts_epilogue(op)) {
        const std::vector<Id> consumers = adj.count(op.id) ? adj[op.id] : std::vector<Id>();
        if (consumers.size() == 1) {
          const Id cid = consumers[0];
          const auto c = std::find_if(current.begin(), current.end(), [&](const Node &n) { return n.id == cid; });
          Json entry;
          size_t need = 0;
          if (c != current.end() && map_to_epilogue(*c, reverse, op.id, fused_into, &entry, &need)) {
            const std::vector<Id> producers = reverse.count(cid) ? reverse[cid] : std::vector<Id>();
            if (producers.size() == need) {
              Node fused = op;
              Json epi = Json::make_arr();
              if (const Json *e = fused.body.find("epilogue")) epi = *e;
              epi.arr.push_back(entry);
              fused.body.set("epilogue", epi);
              next.push_back(fused);
              removed.insert(cid);
              fused_into[cid] = op.id;
              // the merged node's consumers now hang off the producer ...
              const std::vector<Id> onward = adj.count(cid) ? adj[cid] : std::vector<Id>();
              adj[op.id] = onward;
              for (Id o : onward) {
                auto r = reverse.find(o);
                if (r == reverse.end()) continue;
                r->second.erase(std::remove(r->second.begin(), r->second.end(), cid), r->second.end());
                r->second.push_back(op.id);
              }
              // ... and so do its side inputs (BatchNorm parameters, the skip tensor)
              for (Id p : producers)
                if (p != op.id) {
                  adj[p].push_back(op.id);
                  reverse[op.id].push_back(p);
                }
              modified = true;
              merged = true;
            }
          }
        }
      }
      if (!merged) next.push_back(op);
    }
    current.swap(next);
  }

  // A skip tensor named by a ResidualAdd entry may itself have been merged away in a later
  // sweep (in a chain of residual blocks, the ReLU that ends block i is the skip input of
  // block i+1 and is absorbed by block i's last convolution one sweep after block i+1
  // recorded it).  The reference leaves the stale id in place (src/core/optimizer.rs:139-147
  // resolves only at the time of the merge); an id that names no node cannot be executed,
  // so it is resolved here to the node that now produces that tensor.
  for (Node &n : current) {
    if (removed.count(n.id)) continue;
    Json *epi = nullptr;
    for (auto &kv : n.body.obj)
      if (kv.first == "epilogue") epi = &kv.second;
    if (epi == nullptr || epi->type != Json::Array) continue;
    for (Json &e : epi->arr) {
      if (e.type != Json::Object || e.obj.size() != 1 || e.obj[0].first != "ResidualAdd") continue;
      for (auto &f : e.obj[0].second.obj)
        if (f.first == "residual_ptr" && f.second.type == Json::Number) {
          Id skip = (Id)f.second.num;
          for (auto it = fused_into.find(skip); it != fused_into.end(); it = fused_into.find(skip)) skip = it->second;
          f.second = Json::make_num((double)skip);
        }
    }
  }

  Json ops_out = Json::make_arr();
  for (const Node &n : current) {
    if (removed.count(n.id)) continue;
    Json j = Json::make_obj();
    j.set(n.kind, n.body);
    ops_out.arr.push_back(j);
  }
  std::set<std::pair<Id, Id>> deps;
  for (const auto &kv : adj) {
    if (removed.count(kv.first)) continue;
    for (Id dst : kv.second)
      if (!removed.count(dst)) deps.insert({kv.first, dst});
  }
  Json deps_out = Json::make_arr();
  for (const auto &d : deps) {
    Json pair = Json::make_arr();
    pair.arr.push_back(Json::make_num((double)d.first));
    pair.arr.push_back(Json::make_num((double)d.second));
    deps_out.arr.push_back(pair);
  }
  graph->set("operators", ops_out);
  graph->set("dependencies", deps_out);
  return true;
}

}  // namespace tracea_amd
