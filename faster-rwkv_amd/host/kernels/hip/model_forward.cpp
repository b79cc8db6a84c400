// model_forward / model_forward_seq for Device::kHIP.
//
// One token of RWKV-4 is 4 fused launches per layer plus gather and head (98 for a
// 24-layer model, against ~415 in kernels/default/model_forward.cpp:105-188 over
// kernels/cuda).  All buffers are fixed for the life of the model, so the whole token is
// captured once into a HIP graph and replayed.  The token-shift states ping-pong between
// two buffers (the kernel that writes the new state runs while other workgroups still read
// the old one), hence one graph per parity.  The token id reaches the first kernel through a
// small ring in pinned host memory, and the head kernel stores the logits to pinned host memory as
// well as to device memory, so a step costs the host one graph launch and one stream wait.  The recurrent state that model code sees
// (Model::states()) is kept as views of these buffers; states assigned from outside
// (ResetStates, LoadStateFile, set_states) are copied in on the next call.
//
// A greedy loop (GreedyDecode, behind fr_greedy_decode) does not need the host between two tokens:
// a second set of graphs starts with a kernel that picks the token from the arg-max pairs the previous
// token left behind, so the tokens are queued back to back and the host waits once per batch.
//
// FR_HIP_GENERIC=1 selects the operator-by-operator loops (one token and seq mode) instead; FR_HIP_NO_GRAPH=1 keeps
// the fused path but launches eagerly.
#include <algorithm>
#include <cstdlib>
#include <cmath>
#include <cstring>

#include "kernels/hip/context.h"
#include "kernels/hip/hip_model.h"
#include "kernels/kernels.h"
#include "kernels/registry.h"
#include "model.h"

namespace rwkv {
namespace hip {

struct DecodePlan {
  static constexpr int kRing = 64;
  static constexpr int kArgmaxBlocks = 64;
  int L = 0, C = 0, F = 0, V = 0, n_logits = 0;
  Tensor x, ws, counter;
  Tensor logits_dev;
  Tensor pairs_dev[2];                         // the arg-max pairs of the step on parity 0 / 1, for the device-side greedy loop
  float *logits_host[2] = {nullptr, nullptr};  // pinned; the head kernel stores the logits here too, the arg-max pairs follow
  int32_t *ring = nullptr;                     // pinned; token ids, read by the first kernel
  uint32_t fed = 0;                            // tokens fed so far == the device counter
  bool v5 = false;                      // RWKV-5.x: state is (shift, [H,S,S] matrix, shift)
  bool v50 = false;                     // RWKV-5.0: no gate, 13 attention parameters
  int H = 0;
  std::vector<Tensor> aa, bb, pp;       // RWKV-4
  std::vector<Tensor> wkv;              // RWKV-5
  std::vector<Tensor> sx_att[2], sx_ffn[2];
  // the state tensors model code sees for shift-state side `side`: (layer, index) -> the plan's buffer
  Tensor &view(int side, int l, size_t j) {
    if (j == 0) return sx_att[side][l];
    if (v5) return j == 1 ? wkv[l] : sx_ffn[side][l];
    return j == 1 ? aa[l] : j == 2 ? bb[l] : j == 3 ? pp[l] : sx_ffn[side][l];
  }
  size_t n_state() const { return v5 ? 3 : 5; }
  int parity = 0;                             // which ping-pong side holds the current shift states
  frhip_graph graph[2] = {nullptr, nullptr};
  // greedy loop kept on the device (GreedyDecode): the same token, but its first kernel takes the token
  // from the previous step's arg-max pairs and notes it in `chain_ids` (pinned) for the host
  static constexpr int kChainIds = 1024;
  frhip_graph chain[2] = {nullptr, nullptr};
  frhip_graph chain_block = nullptr;  // chain_block_len (even) chained tokens starting on parity 0, as one graph
  int chain_block_len = 2;            // FR_HIP_CHAIN_BLOCK: 2 measured best (4, 8: 0.7 % slower; 16, 32: 1.5-3 % slower)
  int32_t *chain_ids = nullptr;
  bool use_graph = true;
  bool owned_logits = false;  // FR_HIP_OWNED_LOGITS: Run() returns a tensor of its own instead of a view of the pinned ring
  ~DecodePlan() {
    for (auto g : graph)
      if (g) frhip_graph_destroy(g);
    for (auto g : chain)
      if (g) frhip_graph_destroy(g);
    if (chain_block) frhip_graph_destroy(chain_block);
    if (ring) frhip_host_free(ring);
    if (chain_ids) frhip_host_free(chain_ids);
    for (auto h : logits_host)
      if (h) frhip_host_free(h);
  }
};

static void alloc_state_buffers(DecodePlan &p) {
  const int C = p.C;
  const Device d = Device::kHIP;
  p.aa.clear(), p.bb.clear(), p.pp.clear(), p.wkv.clear();
  for (int s = 0; s < 2; s++) p.sx_att[s].clear(), p.sx_ffn[s].clear();
  for (int l = 0; l < p.L; l++) {
    if (p.v5) {
      p.wkv.push_back(Tensor::Empty({p.H, C / p.H, C / p.H}, DType::kFloat32, d));
    } else {
      p.aa.push_back(Tensor::Empty({C}, DType::kFloat32, d));
      p.bb.push_back(Tensor::Empty({C}, DType::kFloat32, d));
      p.pp.push_back(Tensor::Empty({C}, DType::kFloat32, d));
    }
    for (int s = 0; s < 2; s++) {
      p.sx_att[s].push_back(Tensor::Empty({C}, DType::kFloat16, d));
      p.sx_ffn[s].push_back(Tensor::Empty({C}, DType::kFloat16, d));
    }
  }
}

static std::shared_ptr<DecodePlan> make_plan(Model *model, ModelExtra &ex) {
  auto p = std::make_shared<DecodePlan>();
  p->L = model->n_layer();
  p->C = model->n_embd();
  p->v5 = model->version() != "4";
  p->v50 = model->version() == "5";
  p->H = model->head_size();
  p->F = model->n_ffn() > 0 ? model->n_ffn() : static_cast<int>(model->_params[15].size(1));
  p->V = static_cast<int>(ex.emb_table.size(0));
  const int C = p->C;
  const Device d = Device::kHIP;
  p->x = Tensor::Empty({C}, DType::kFloat16, d);
  p->ws = Tensor::Empty({static_cast<LengthType>(frhip_decode_workspace_bytes(C, p->F))}, DType::kInt8, d);
  p->counter = Tensor::Empty({1}, DType::kInt32, d);
  FRHIP_CHECK(frhip_fill(p->counter.data_ptr(), FRHIP_F32, 0.0f, 1, stream()));  // all-zero bits
  p->n_logits = static_cast<int>(model->_params.back().size(1));
  p->logits_dev = Tensor::Empty({p->n_logits}, DType::kFloat32, d);
  for (auto &pd : p->pairs_dev) {
    pd = Tensor::Empty({2 * DecodePlan::kArgmaxBlocks}, DType::kFloat32, d);
    FRHIP_CHECK(frhip_fill(pd.data_ptr(), FRHIP_F32, 0.0f, 2 * DecodePlan::kArgmaxBlocks, stream()));
  }
  void *h = nullptr;
  FRHIP_CHECK(frhip_host_malloc(&h, sizeof(int32_t) * DecodePlan::kRing));
  p->ring = static_cast<int32_t *>(h);
  FRHIP_CHECK(frhip_host_malloc(&h, sizeof(int32_t) * DecodePlan::kChainIds));
  p->chain_ids = static_cast<int32_t *>(h);
  for (auto &lh : p->logits_host) {
    FRHIP_CHECK(frhip_host_malloc(&h, sizeof(float) * (static_cast<size_t>(p->n_logits) + 2 * DecodePlan::kArgmaxBlocks)));
    lh = static_cast<float *>(h);
  }
  alloc_state_buffers(*p);
  p->use_graph = std::getenv("FR_HIP_NO_GRAPH") == nullptr;  // fixed when the model first runs
  p->owned_logits = std::getenv("FR_HIP_OWNED_LOGITS") != nullptr;
  if (const char *e = std::getenv("FR_HIP_CHAIN_BLOCK")) p->chain_block_len = std::atoi(e) / 2 * 2;  // 0: token by token
  return p;
}

// The fused path updates the recurrent state in place, in buffers the plan owns, and Model::states()
// hands out those buffers.  The reference's operators return fresh tensors every step
// (kernels/cuda/att.cu:344-353), so a caller may keep a copy of states() as a snapshot and give it back
// to set_states() later.  To keep that working, a buffer that someone outside still holds (a copy of the
// States vector shares its storage) is never written again: the plan moves to fresh buffers that start
// with the current contents, and the captured graphs, which name the old addresses, are dropped.
static void detach_if_snapshotted(Model *model, DecodePlan &p) {
  auto &st = model->states();
  bool held = false;
  for (int l = 0; l < p.L && !held; l++)
    for (int side = 0; side < 2 && !held; side++)
      for (size_t j = 0; j < p.n_state(); j++) {
        if (side == 1 && j != 0 && j != p.n_state() - 1) continue;  // aa, bb, pp / wkv exist once
        Tensor &b = p.view(side, l, j);
        const long expected = 1 + (st[l][j].shares_storage_with(b) ? 1 : 0);
        if (b.storage_use_count() > expected) {
          held = true;
          break;
        }
      }
  if (!held) return;
  DecodePlan old;  // keeps the old buffers alive until their contents are copied
  old.v5 = p.v5;
  old.aa = p.aa, old.bb = p.bb, old.pp = p.pp, old.wkv = p.wkv;
  for (int s = 0; s < 2; s++) old.sx_att[s] = p.sx_att[s], old.sx_ffn[s] = p.sx_ffn[s];
  alloc_state_buffers(p);
  for (int l = 0; l < p.L; l++)
    for (size_t j = 0; j < p.n_state(); j++) {
      Tensor &src = old.view(p.parity, l, j), &dst = p.view(p.parity, l, j);
      FRHIP_CHECK(frhip_memcpy_async(dst.data_ptr(), src.data_ptr(), src.nbytes(), FRHIP_D2D, stream()));
      if (st[l][j].shares_storage_with(src)) st[l][j] = dst;
    }
  FRHIP_CHECK(frhip_stream_sync(stream()));
  for (auto *set : {p.graph, p.chain})
    for (int i = 0; i < 2; i++) {
      if (set[i]) frhip_graph_destroy(set[i]);
      set[i] = nullptr;
    }
  if (p.chain_block) frhip_graph_destroy(p.chain_block);
  p.chain_block = nullptr;
}

// Bring states assigned from outside into the plan's buffers and rebind the model's
// state tensors to them.
static void adopt_states(Model *model, DecodePlan &p) {
  auto &st = model->states();
  RV_CHECK(static_cast<int>(st.size()) == p.L);
  for (int l = 0; l < p.L; l++) {
    RV_CHECK(st[l].size() == p.n_state());
    for (size_t j = 0; j < p.n_state(); j++) {
      Tensor &mine = p.view(p.parity, l, j);
      if (st[l][j].data_ptr() == mine.data_ptr()) continue;
      RV_CHECK(st[l][j].nbytes() == mine.nbytes() && st[l][j].dtype() == mine.dtype())
          << "state " << l << "/" << j << " has the wrong shape or dtype";
      Tensor src = st[l][j].device() == Device::kHIP ? st[l][j] : Copy(st[l][j], Device::kHIP);
      FRHIP_CHECK(frhip_memcpy_async(mine.data_ptr(), src.data_ptr(), src.nbytes(), FRHIP_D2D, stream()));
      if (src.data_ptr() != st[l][j].data_ptr()) FRHIP_CHECK(frhip_stream_sync(stream()));  // src dies here
      st[l][j] = mine;
    }
  }
}

// `chained`: the token comes from the arg-max pairs the previous step left in device memory (pairs_dev)
// (that step ran on the other parity) instead of from the host's ring.
static void issue_token(Model *model, ModelExtra &ex, DecodePlan &p, bool chained = false) {
  const auto &P = model->_params;
  frhip_stream s = stream();
  const int C = p.C, F = p.F;
  const int cur = p.parity, nxt = 1 - p.parity;
  if (chained)
    FRHIP_CHECK(frhip_embed_argmax(ex.emb_table.data_ptr(), p.V, 2 * C, p.pairs_dev[nxt].data_ptr(),
                                   DecodePlan::kArgmaxBlocks, p.chain_ids, DecodePlan::kChainIds,
                                   reinterpret_cast<uint32_t *>(p.counter.data_ptr()), p.x.data_ptr(), s));
  else
    FRHIP_CHECK(frhip_embed_ring(ex.emb_table.data_ptr(), p.V, 2 * C, p.ring, DecodePlan::kRing,
                                 reinterpret_cast<uint32_t *>(p.counter.data_ptr()), p.x.data_ptr(), s));
  size_t pi = 0;
  for (int l = 0; l < p.L && p.v50; l++) {
    const frhip_weight *kw = find_weight(P[pi + 9]), *vw = find_weight(P[pi + 10]), *rw = find_weight(P[pi + 11]),
                       *ow = find_weight(P[pi + 12]);
    RV_CHECK(kw && vw && rw && ow);
    FRHIP_CHECK(frhip_att_one_v5(C, p.H, p.x.data_ptr(), p.sx_att[cur][l].data_ptr(), p.wkv[l].data_ptr<float>(),
                                 P[pi].data_ptr(), P[pi + 1].data_ptr(), P[pi + 2].data_ptr<float>(),
                                 P[pi + 3].data_ptr<float>(), P[pi + 4].data_ptr(), P[pi + 5].data_ptr(),
                                 P[pi + 6].data_ptr(), P[pi + 7].data_ptr<float>(), P[pi + 8].data_ptr<float>(), kw,
                                 vw, rw, ow, p.x.data_ptr(), p.sx_att[nxt][l].data_ptr(), p.wkv[l].data_ptr<float>(),
                                 p.ws.data_ptr(), s));
    pi += 13;
    const frhip_weight *fk = find_weight(P[pi + 4]), *fv = find_weight(P[pi + 5]), *frw = find_weight(P[pi + 6]);
    RV_CHECK(fk && fv && frw);
    FRHIP_CHECK(frhip_ffn_one(C, F, p.x.data_ptr(), p.sx_ffn[cur][l].data_ptr(), P[pi].data_ptr(),
                              P[pi + 1].data_ptr(), P[pi + 2].data_ptr(), P[pi + 3].data_ptr(), fk, fv, frw,
                              p.x.data_ptr(), p.sx_ffn[nxt][l].data_ptr(), (l + 1) % 6 == 0 ? 1 : 0, p.ws.data_ptr(),
                              s));
    pi += 7;
  }
  for (int l = 0; l < p.L && p.v5 && !p.v50; l++) {
    const frhip_weight *kw = find_weight(P[pi + 10]), *vw = find_weight(P[pi + 11]), *rw = find_weight(P[pi + 12]),
                       *gw = find_weight(P[pi + 13]), *ow = find_weight(P[pi + 14]);
    RV_CHECK(kw && vw && rw && gw && ow);
    FRHIP_CHECK(frhip_att_one_v5_1(C, p.H, p.x.data_ptr(), p.sx_att[cur][l].data_ptr(), p.wkv[l].data_ptr<float>(),
                                   P[pi].data_ptr(), P[pi + 1].data_ptr(), P[pi + 2].data_ptr<float>(),
                                   P[pi + 3].data_ptr<float>(), P[pi + 4].data_ptr(), P[pi + 5].data_ptr(),
                                   P[pi + 6].data_ptr(), P[pi + 7].data_ptr(), P[pi + 8].data_ptr<float>(),
                                   P[pi + 9].data_ptr<float>(), kw, vw, rw, gw, ow, p.x.data_ptr(),
                                   p.sx_att[nxt][l].data_ptr(), p.wkv[l].data_ptr<float>(), p.ws.data_ptr(), s));
    pi += 15;
    const frhip_weight *fk = find_weight(P[pi + 4]), *fv = find_weight(P[pi + 5]), *frw = find_weight(P[pi + 6]);
    RV_CHECK(fk && fv && frw);
    FRHIP_CHECK(frhip_ffn_one(C, F, p.x.data_ptr(), p.sx_ffn[cur][l].data_ptr(), P[pi].data_ptr(),
                              P[pi + 1].data_ptr(), P[pi + 2].data_ptr(), P[pi + 3].data_ptr(), fk, fv, frw,
                              p.x.data_ptr(), p.sx_ffn[nxt][l].data_ptr(), (l + 1) % 6 == 0 ? 1 : 0, p.ws.data_ptr(),
                              s));
    pi += 7;
  }
  for (int l = 0; l < p.L && !p.v5; l++) {
    const frhip_weight *kw = find_weight(P[pi + 7]), *vw = find_weight(P[pi + 8]), *rw = find_weight(P[pi + 9]),
                       *ow = find_weight(P[pi + 10]);
    RV_CHECK(kw && vw && rw && ow);
    FRHIP_CHECK(frhip_att_one_v4(C, p.x.data_ptr(), p.sx_att[cur][l].data_ptr(), p.aa[l].data_ptr<float>(),
                                 p.bb[l].data_ptr<float>(), p.pp[l].data_ptr<float>(), P[pi].data_ptr(),
                                 P[pi + 1].data_ptr(), P[pi + 2].data_ptr(), P[pi + 3].data_ptr(),
                                 P[pi + 4].data_ptr(), P[pi + 5].data_ptr<float>(), P[pi + 6].data_ptr<float>(), kw,
                                 vw, rw, ow, p.x.data_ptr(), p.sx_att[nxt][l].data_ptr(), p.aa[l].data_ptr<float>(),
                                 p.bb[l].data_ptr<float>(), p.pp[l].data_ptr<float>(), p.ws.data_ptr(), s));
    pi += 11;
    const frhip_weight *fk = find_weight(P[pi + 4]), *fv = find_weight(P[pi + 5]), *frw = find_weight(P[pi + 6]);
    RV_CHECK(fk && fv && frw);
    FRHIP_CHECK(frhip_ffn_one(C, F, p.x.data_ptr(), p.sx_ffn[cur][l].data_ptr(), P[pi].data_ptr(),
                              P[pi + 1].data_ptr(), P[pi + 2].data_ptr(), P[pi + 3].data_ptr(), fk, fv, frw,
                              p.x.data_ptr(), p.sx_ffn[nxt][l].data_ptr(), (l + 1) % 6 == 0 ? 1 : 0, p.ws.data_ptr(),
                              s));
    pi += 7;
  }
  const frhip_weight *hw = find_weight(P[pi + 2]);
  RV_CHECK(hw != nullptr);
  // The head stores every logit twice: to device memory, where the greedy sampler's step (Sampler::Sample
  // with top_k = 1, sampler.cpp:28-32) reads them, and to the pinned host buffer the call returns, so that
  // they cross the bus while the product runs; the per-slice pairs of the arg-max go to the host directly.
  // A caller that only wants the most likely token need not read 4 * V bytes of fresh host memory.
  FRHIP_CHECK(frhip_head_mirror(C, p.x.data_ptr(), P[pi].data_ptr(), P[pi + 1].data_ptr(), hw,
                                p.logits_dev.data_ptr<float>(), p.logits_host[cur], s));
  // the pairs twice: in device memory for a next step that picks its own token, beside the host's logits for the host
  FRHIP_CHECK(frhip_argmax_blocks_f32_mirror(p.logits_dev.data_ptr<float>(), p.n_logits, p.pairs_dev[cur].data_ptr(),
                                             p.logits_host[cur] + p.n_logits, DecodePlan::kArgmaxBlocks, s));
}

// Captures `count` consecutive tokens, the first on parity `parity`, as one graph; nothing runs, and the
// plan is left as it was.
static frhip_graph capture_tokens(Model *model, ModelExtra &ex, DecodePlan &p, int parity, bool chained, int count) {
  frhip_stream s = stream();
  const int saved = p.parity;
  frhip_graph g = nullptr;
  FRHIP_CHECK(frhip_graph_begin(s));
  try {
    p.parity = parity;
    for (int k = 0; k < count; k++) {
      issue_token(model, ex, p, chained);
      p.parity = 1 - p.parity;
    }
  } catch (...) {
    p.parity = saved;
    frhip_graph_end(s, &g);
    if (g) frhip_graph_destroy(g);
    throw;
  }
  p.parity = saved;
  FRHIP_CHECK(frhip_graph_end(s, &g));
  return g;
}

// Every graph the plan can replay is captured the first time one of its kind is needed, both parities
// at once, so that no later call pays for a capture because of the parity it happens to start on.
static void ensure_graphs(Model *model, ModelExtra &ex, DecodePlan &p, bool chained) {
  if (!p.use_graph) return;
  for (int side = 0; side < 2; side++) {
    frhip_graph &g = chained ? p.chain[side] : p.graph[side];
    if (!g) g = capture_tokens(model, ex, p, side, chained, 1);
  }
  if (chained && p.chain_block_len >= 2 && !p.chain_block)
    p.chain_block = capture_tokens(model, ex, p, 0, true, p.chain_block_len);
}

// Replays the graph of one token on the current parity and moves the plan on to the next token; does
// not wait.
static void launch_token(Model *model, ModelExtra &ex, DecodePlan &p, bool chained) {
  const int cur = p.parity;
  if (!p.use_graph) {
    issue_token(model, ex, p, chained);
  } else {
    ensure_graphs(model, ex, p, chained);
    FRHIP_CHECK(frhip_graph_launch(chained ? p.chain[cur] : p.graph[cur], stream()));
  }
  p.fed++;  // the device counter advances when the first kernel of the step runs
  p.parity = 1 - cur;
}

// chain_block_len chained tokens in one graph (the gap between two graph launches on a stream is paid
// once per block instead of once per token).  The plan must be on parity 0; it is again afterwards.
static void launch_chain_block(Model *model, ModelExtra &ex, DecodePlan &p) {
  RV_CHECK(p.parity == 0 && p.chain_block_len % 2 == 0);
  ensure_graphs(model, ex, p, true);
  FRHIP_CHECK(frhip_graph_launch(p.chain_block, stream()));
  p.fed += p.chain_block_len;
}

// After the stream has been waited for: the model's state tensors follow the ping-pong side, and the
// arg-max of the last token's logits (buffer `cur`) is finished on the host.
static void settle(Model *model, ModelExtra &ex, DecodePlan &p, int cur) {
  auto &st = model->states();
  const size_t last = p.v5 ? 2 : 4;
  for (int l = 0; l < p.L; l++) {
    st[l][0] = p.view(p.parity, l, 0);
    st[l][last] = p.view(p.parity, l, last);
  }
  // second step of the arg-max: greater value, then smaller index, over the per-slice pairs
  const float *pairs = p.logits_host[cur] + p.n_logits;
  float best = -INFINITY;
  int32_t idx = p.n_logits;
  for (int b = 0; b < DecodePlan::kArgmaxBlocks; b++) {
    int32_t bi;
    std::memcpy(&bi, pairs + 2 * b + 1, sizeof(bi));
    if (pairs[2 * b] > best || (pairs[2 * b] == best && bi < idx)) {
      best = pairs[2 * b];
      idx = bi;
    }
  }
  ex.last_argmax = idx < p.n_logits ? idx : 0;
  ex.last_argmax_of = p.logits_host[cur];
}

Tensor ModelForward(Model *model, Device device, int id) {
  const bool generic = std::getenv("FR_HIP_GENERIC") != nullptr;  // read per call so that one process can compare both paths
  const std::string &ver = model->version();
  if (generic || !(ver == "4" || ver == "5" || ver == "5.1" || ver == "5.2")) return def::ModelForward(model, device, id);
  auto ex = extra_of(model);
  if (!ex->plan) ex->plan = make_plan(model, *ex);
  DecodePlan &p = *ex->plan;
  RV_CHECK(id >= 0 && id < p.V) << "token id " << id << " out of range";
  detach_if_snapshotted(model, p);
  adopt_states(model, p);
  // every call ends with a stream synchronisation, so the device has consumed all earlier slots
  p.ring[p.fed % DecodePlan::kRing] = id;
  const int cur = p.parity;
  launch_token(model, *ex, p, false);
  // The head kernel has stored the logits into pinned host memory; waiting for the stream
  // is the step's one synchronisation point (the reference's is the blocking cudaMemcpy in
  // tensor.cpp:65-68).  The returned CPU tensor is a view, valid until the next-but-one call.
  FRHIP_CHECK(frhip_stream_sync(stream()));
  settle(model, *ex, p, cur);
  if (p.owned_logits) {  // a tensor of the caller's own, as the reference returns (model.cpp:179-186)
    Tensor out = Tensor::Empty({p.n_logits}, DType::kFloat32, Device::kCPU);
    std::memcpy(out.data_ptr(), p.logits_host[cur], sizeof(float) * static_cast<size_t>(p.n_logits));
    ex->last_argmax_of = out.data_ptr();
    return out;
  }
  return Tensor::FromPtr(p.logits_host[cur], {p.n_logits}, DType::kFloat32, Device::kCPU);
}

// `steps` greedy tokens starting from `first_id` with the host out of the loop: after the first token
// (an ordinary ModelForward) every step's first kernel picks its token from the arg-max pairs of the step
// before it, so the graphs are queued back to back and the host waits once per batch of at most
// kChainIds - 1 steps instead of once per token (the top_k = 1 case of chat.cpp:56-92, where the host
// sits between two forward passes).  The tokens, the logits of the last step and the state left behind
// are those of the loop of ModelForward calls.  Returns false, having done nothing, when the fused
// graph path is not the one in use; `last_logits`, if given, receives what the last Run would return.
bool GreedyDecode(Model *model, int first_id, int steps, int *out_ids, Tensor *last_logits) {
  const std::string &ver = model->version();
  if (model->act_device() != Device::kHIP || std::getenv("FR_HIP_GENERIC") || std::getenv("FR_HIP_NO_GRAPH") ||
      std::getenv("FR_HIP_GREEDY_ON_HOST") ||
      !(ver == "4" || ver == "5" || ver == "5.1" || ver == "5.2"))
    return false;
  if (steps <= 0) return true;
  Tensor lg = hip::ModelForward(model, Device::kHIP, first_id);
  auto ex = extra_of(model);
  DecodePlan &p = *ex->plan;
  if (!p.use_graph) {  // the plan was made under FR_HIP_NO_GRAPH: finish token by token
    out_ids[0] = ex->last_argmax;
    for (int i = 1; i < steps; i++) {
      lg = hip::ModelForward(model, Device::kHIP, out_ids[i - 1]);
      out_ids[i] = ex->last_argmax;
    }
    if (last_logits) *last_logits = lg;
    return true;
  }
  out_ids[0] = ex->last_argmax;
  int done = 1;
  while (done < steps) {
    const int n = std::min(steps - done, DecodePlan::kChainIds - 1);
    const uint32_t fed0 = p.fed;
    int cur = p.parity;  // parity of the last token launched
    int k = 0;
    auto one = [&]() {
      cur = p.parity;
      launch_token(model, *ex, p, true);
      k++;
    };
    if (p.chain_block_len >= 2) {
      if (p.parity == 1 && k < n) one();
      while (n - k >= p.chain_block_len) {
        launch_chain_block(model, *ex, p);
        cur = 1;
        k += p.chain_block_len;
      }
    }
    while (k < n) one();
    FRHIP_CHECK(frhip_stream_sync(stream()));
    // step done + k was fed the token out_ids[done + k - 1] and noted it in slot (fed0 + k)
    for (int k = 1; k < n; k++) out_ids[done + k - 1] = p.chain_ids[(fed0 + k) % DecodePlan::kChainIds];
    settle(model, *ex, p, cur);
    out_ids[done + n - 1] = ex->last_argmax;
    done += n;
    if (last_logits) {
      if (p.owned_logits) {
        Tensor out = Tensor::Empty({p.n_logits}, DType::kFloat32, Device::kCPU);
        std::memcpy(out.data_ptr(), p.logits_host[cur], sizeof(float) * static_cast<size_t>(p.n_logits));
        ex->last_argmax_of = out.data_ptr();
        lg = out;
      } else {
        lg = Tensor::FromPtr(p.logits_host[cur], {p.n_logits}, DType::kFloat32, Device::kCPU);
      }
    }
  }
  if (last_logits) *last_logits = lg;
  return true;
}

// Index of the largest logit of the tensor `logits` if that tensor is the one the last one-token
// forward pass of `model` returned and the pass computed the index on the device.
bool device_argmax(Model *model, const Tensor &logits, int *id) {
  auto ex = extra_of(model);
  if (!ex || ex->last_argmax_of == nullptr || ex->last_argmax_of != logits.data_ptr()) return false;
  *id = ex->last_argmax;
  return true;
}

// Seq mode (reference: kernels/default/model_forward_seq.cpp:48-184): embedding rows are
// gathered on the device, every layer runs its seq operator over all T rows (MFMA products,
// chunked WKV scans), and only the last row goes through ln_out and the head (all rows with
// full_output).  RWKV-4, which
// upstream cannot run in seq mode (:111-112), goes through the `att_seq` operator.
// FR_HIP_SEQ_FALLBACK=1 selects the loop of one-token steps (:34-46) instead.
Tensor ModelForwardSeq(Model *model, Device device, const std::vector<int> &ids, bool full_output) {
  const std::string &ver = model->version();
  if (std::getenv("FR_HIP_SEQ_FALLBACK") || !(ver == "4" || ver == "5" || ver == "5.2"))
    return def::ModelForwardSeqFallback(model, device, ids, full_output);
  // the reference-shaped operator loop (vgather, seq operators, slice, layernorm, matmul, cast_dtype)
  if (std::getenv("FR_HIP_GENERIC")) return def::ModelForwardSeq(model, device, ids, full_output);
  RV_CHECK(!ids.empty());
  // A prompt of two or three tokens is quicker as one-token steps (0.7 ms each for the 1.5B shape) than as a pass
  // of the seq operators, which for so few rows costs its ~290 launches (1.9 ms); FR_HIP_SEQ_ALWAYS=1: never.
  if (!full_output && ids.size() < 4 && !std::getenv("FR_HIP_SEQ_ALWAYS")) {
    Tensor out;
    for (int id : ids) out = hip::ModelForward(model, device, id);
    // the one-token result is a view of the plan's pinned ring (valid until the next-but-one call); a prompt's
    // result belongs to the caller, as the seq operators' does
    Tensor owned = Tensor::Empty(out.shape(), out.dtype(), Device::kCPU);
    std::memcpy(owned.data_ptr(), out.data_ptr(), out.nbytes());
    return owned;
  }
  auto ex = extra_of(model);
  const int T = static_cast<int>(ids.size()), C = model->n_embd();
  const int V = static_cast<int>(ex->emb_table.size(0));
  for (int id : ids) RV_CHECK(id >= 0 && id < V) << "token id " << id << " out of range";
  frhip_stream s = stream();
  // ids -> device -> gather (reference: vgather, T separate device copies)
  Tensor ids_cpu = Tensor::Empty({T}, DType::kInt32, Device::kCPU);
  std::memcpy(ids_cpu.data_ptr(), ids.data(), sizeof(int32_t) * ids.size());
  Tensor ids_dev = Copy(ids_cpu, Device::kHIP, true);
  Tensor x = Tensor::Empty({T, C}, DType::kFloat16, Device::kHIP);
  FRHIP_CHECK(frhip_gather_rows(ex->emb_table.data_ptr(), ids_dev.data_ptr<int32_t>(), x.data_ptr(), T, 2 * C, s));

  auto &states = model->states();
  const auto &p = model->_params;
  size_t pi = 0;
  for (size_t i = 0; i < states.size(); i++) {
    auto &st = states[i];
    if (ver == "4") {
      std::tie(x, st[0], st[1], st[2], st[3]) =
          att_seq(x, st[0], st[1], st[2], st[3], p[pi], p[pi + 1], p[pi + 2], p[pi + 3], p[pi + 4], p[pi + 5],
                  p[pi + 6], p[pi + 7], p[pi + 8], p[pi + 9], p[pi + 10]);
      pi += 11;
    } else if (ver == "5") {
      std::tie(x, st[0], st[1]) =
          att_seq_v5(x, st[0], st[1], p[pi], p[pi + 1], p[pi + 2], p[pi + 3], p[pi + 4], p[pi + 5], p[pi + 6],
                     p[pi + 7], p[pi + 8], p[pi + 9], p[pi + 10], p[pi + 11], p[pi + 12]);
      pi += 13;
    } else {
      std::tie(x, st[0], st[1]) =
          att_seq_v5_2(x, st[0], st[1], p[pi], p[pi + 1], p[pi + 2], p[pi + 3], p[pi + 4], p[pi + 5], p[pi + 6],
                       p[pi + 7], p[pi + 8], p[pi + 9], p[pi + 10], p[pi + 11], p[pi + 12], p[pi + 13], p[pi + 14],
                       model->n_att());
      pi += 15;
    }
    const int off = ver[0] == '5' ? 2 : 4;
    // the halving after every sixth layer (model_forward_seq.cpp:163-165) rides in the ffn's last epilogue
    std::tie(x, st[off]) = ffn_seq_div2(x, st[off], p[pi], p[pi + 1], p[pi + 2], p[pi + 3], p[pi + 4], p[pi + 5],
                                        p[pi + 6], (i + 1) % 6 == 0);
    pi += 7;
  }
  const frhip_weight *hw = find_seq_weight(p[pi + 2], full_output ? T : 1);
  RV_CHECK(hw != nullptr);
  if (full_output) {
    // every row -> ln_out -> head -> fp32 [T, V] (model_forward_seq.cpp:173-178 without the slice)
    Tensor y = layernorm(x, p[pi], p[pi + 1]);
    Tensor lg = Tensor::Empty({T, static_cast<LengthType>(hw->N)}, DType::kFloat16, Device::kHIP);
    FRHIP_CHECK(frhip_gemm(y.data_ptr(), hw, lg.data_ptr(), T, FRHIP_F16, s));
    return cast_dtype(lg, DType::kFloat32);
  }
  // last row -> ln_out -> head -> fp32 (model_forward_seq.cpp:170-178)
  Tensor logits = Tensor::Empty({static_cast<LengthType>(hw->N)}, DType::kFloat32, Device::kHIP);
  const char *last = static_cast<const char *>(x.data_ptr()) + static_cast<size_t>(T - 1) * C * 2;
  FRHIP_CHECK(frhip_head(C, last, p[pi].data_ptr(), p[pi + 1].data_ptr(), hw, logits.data_ptr<float>(), s));
  return logits;
}

KernelRegister model_forward_reg("model_forward", Device::kHIP, ModelForward);
KernelRegister model_forward_seq_reg("model_forward_seq", Device::kHIP, ModelForwardSeq);

}  // namespace hip
}  // namespace rwkv
