// The torch operator layer over the C ABI of include/pplx_a2a.h.
//
// Takes the place of the reference's csrc/bindings/all_to_all_ops.cpp (create / destroy /
// dispatch / combine ops, tensor checks, stride extraction) and csrc/bindings/bindings.cpp
// (TORCH_LIBRARY(pplx_kernels)).  The ops keep the reference's names and schemas
// (csrc/bindings/all_to_all_ops.cpp:329-391), so torch.compile traces a step through the
// dispatcher and its Meta kernels.  The same entry points are also exported as plain CPython
// functions (module pplx_kernels._C): an eager per-rank call made through them costs no trip
// through the op dispatcher, which matters because a step of R simulated ranks is 2 R calls.
//
// What differs from the reference follows from the loopback: `group_name` resolves to a
// process-local world (the reference resolves a c10d process group and exchanges IPC handles,
// csrc/bindings/all_to_all_ops.cpp:79-106), a step is collective over the calls of the world's
// ranks, so the tensors of the calls recorded so far are kept alive here until the step's last
// rank has called, and a failed call is an exception, never an exit.
#include <Python.h>

#include <ATen/core/Tensor.h>
#include <c10/hip/HIPFunctions.h>
#include <c10/hip/HIPStream.h>
#include <c10/util/Exception.h>
#include <torch/csrc/Exceptions.h>
#include <torch/csrc/autograd/python_variable.h>
#include <torch/library.h>

#include <array>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "pplx_a2a.h"

namespace {

using fptr_t = int64_t;

const char *status_name(int status) {
  switch (status) {
    case PPLX_A2A_INVALID_ARGUMENT: return "invalid argument";
    case PPLX_A2A_INVALID_STATE: return "invalid state";
    case PPLX_A2A_HIP_ERROR: return "HIP error";
    case PPLX_A2A_UNSUPPORTED: return "unsupported";
    default: return "error";
  }
}

#define A2A_CHECK(status)                                                                     \
  do {                                                                                        \
    const int st_ = (status);                                                                 \
    TORCH_CHECK(st_ == PPLX_A2A_OK, "pplx_kernels: ", status_name(st_), ": ", pplx_a2a_last_error()); \
  } while (0)

// ---------------------------------------------------------------------------
// Worlds and rank handles
// ---------------------------------------------------------------------------
constexpr int kOps = 2, kModes = 3;  // (dispatch, combine) x (NONE, SEND, RECV)

struct World {
  std::string key;
  pplx_a2a_config_t cfg{};
  pplx_a2a_world_t *ptr = nullptr;
  int handles = 0;
  int split_reserved = -1;  // widest expert_y element split staging was reserved for
  // A step's kernels are enqueued by the last rank to call, so the tensors of the ranks that
  // called earlier are kept alive until then: a temporary such as x.to(device) must not go
  // back to the caching allocator before it has been read.
  std::array<std::vector<std::vector<at::Tensor>>, kOps * kModes> held;
};

struct RankRef {
  World *world;
  uint32_t rank;
};

std::mutex g_mu;  // guards the two maps and every World; held across a call into the library
std::unordered_map<std::string, std::unique_ptr<World>> g_worlds;
std::unordered_map<fptr_t, RankRef> g_ranks;

bool same_config(const pplx_a2a_config_t &a, const pplx_a2a_config_t &b) {
  return a.max_num_tokens == b.max_num_tokens && a.num_experts == b.num_experts &&
         a.experts_per_token == b.experts_per_token && a.world_size == b.world_size &&
         a.dp_size == b.dp_size && a.hidden_dim == b.hidden_dim &&
         a.hidden_dim_bytes == b.hidden_dim_bytes && a.hidden_dim_scale_bytes == b.hidden_dim_scale_bytes;
}

fptr_t create_rank(const std::string &transport, const std::string &group_name, int64_t maxNumTokens,
                   int64_t numExperts, int64_t expertsPerToken, int64_t rank, int64_t worldSize,
                   int64_t dpSize, int64_t hiddenDim, int64_t hiddenDimBytes, int64_t hiddenDimScaleBytes) {
  TORCH_CHECK(maxNumTokens >= 0 && numExperts >= 0 && expertsPerToken >= 0 && worldSize > 0 && dpSize > 0 &&
                  hiddenDim >= 0 && hiddenDimBytes >= 0 && hiddenDimScaleBytes >= 0,
              "pplx_kernels: invalid argument: negative or zero size");
  TORCH_CHECK(rank >= 0, "pplx_kernels: invalid argument: negative rank");
  pplx_a2a_config_t cfg{};
  cfg.max_num_tokens = (uint64_t)maxNumTokens;
  cfg.num_experts = (uint64_t)numExperts;
  cfg.experts_per_token = (uint64_t)expertsPerToken;
  cfg.world_size = (uint32_t)worldSize;
  cfg.dp_size = (uint32_t)dpSize;
  cfg.hidden_dim = (uint64_t)hiddenDim;
  cfg.hidden_dim_bytes = (uint64_t)hiddenDimBytes;
  cfg.hidden_dim_scale_bytes = (uint64_t)hiddenDimScaleBytes;
  TORCH_CHECK(worldSize <= UINT32_MAX && dpSize <= UINT32_MAX && rank <= UINT32_MAX,
              "pplx_kernels: invalid argument: world_size / dp_size / rank out of range");

  const std::string key = transport + ":" + group_name;
  std::lock_guard<std::mutex> lock(g_mu);
  auto it = g_worlds.find(key);
  if (it != g_worlds.end()) {
    TORCH_CHECK(same_config(it->second->cfg, cfg), "pplx_kernels: group '", group_name,
                "' already holds a world with a different configuration; destroy its ranks first or use "
                "another group_name");
  } else {
    auto world = std::make_unique<World>();
    world->key = key;
    world->cfg = cfg;
    // The world lives on the caller's current device (device 0 when no GPU is visible, so that
    // the library reports the missing GPU).
    const int device = c10::hip::device_count() > 0 ? (int)c10::hip::current_device() : 0;
    A2A_CHECK(pplx_a2a_world_create(&cfg, device, &world->ptr));
    for (auto &per_rank : world->held) per_rank.resize(cfg.world_size);
    it = g_worlds.emplace(key, std::move(world)).first;
  }
  World *world = it->second.get();
  pplx_a2a_t *handle = nullptr;
  const int st = pplx_a2a_create(world->ptr, (uint32_t)rank, &handle);
  if (st != PPLX_A2A_OK) {
    const std::string msg = pplx_a2a_last_error();
    if (world->handles == 0) {
      (void)pplx_a2a_world_destroy(world->ptr);
      g_worlds.erase(it);
    }
    TORCH_CHECK(false, "pplx_kernels: ", status_name(st), ": ", msg);
  }
  ++world->handles;
  g_ranks[(fptr_t)handle] = RankRef{world, (uint32_t)rank};
  return (fptr_t)handle;
}

void release_held(World &world, uint32_t rank) {
  for (auto &per_rank : world.held) per_rank[rank].clear();
}

// csrc/bindings/all_to_all_ops.cpp:108
void destroy(fptr_t ptr) {
  std::lock_guard<std::mutex> lock(g_mu);
  auto it = g_ranks.find(ptr);
  TORCH_CHECK(it != g_ranks.end(), "pplx_kernels: unknown all-to-all handle ", ptr);
  World *world = it->second.world;
  // (a handle that leaves in the middle of a step takes its half-made calls along)
  release_held(*world, it->second.rank);
  g_ranks.erase(it);
  A2A_CHECK(pplx_a2a_destroy((pplx_a2a_t *)ptr));
  if (--world->handles == 0) {
    const int st = pplx_a2a_world_destroy(world->ptr);
    const std::string msg = st ? pplx_a2a_last_error() : "";
    const std::string key = world->key;
    g_worlds.erase(key);
    TORCH_CHECK(st == PPLX_A2A_OK, "pplx_kernels: ", status_name(st), ": ", msg);
  }
}

// Interpreter exit: everything is released while the HIP runtime is still up.
void destroy_all() {
  std::lock_guard<std::mutex> lock(g_mu);
  for (auto &entry : g_ranks) (void)pplx_a2a_destroy((pplx_a2a_t *)entry.first);
  g_ranks.clear();
  for (auto &entry : g_worlds) (void)pplx_a2a_world_destroy(entry.second->ptr);
  g_worlds.clear();
}

fptr_t create_intranode(int64_t maxNumTokens, int64_t numExperts, int64_t expertsPerToken, int64_t rank,
                        int64_t worldSize, int64_t dpSize, int64_t hiddenDim, int64_t hiddenDimBytes,
                        int64_t hiddenDimScaleBytes, const std::string &group_name) {
  return create_rank("intranode", group_name, maxNumTokens, numExperts, expertsPerToken, rank, worldSize, dpSize,
                     hiddenDim, hiddenDimBytes, hiddenDimScaleBytes);
}

// One HBM has no second transport: the internode constructor attaches to a loopback world of
// its own and runs the same kernels.
fptr_t create_internode(int64_t maxNumTokens, int64_t numExperts, int64_t expertsPerToken, int64_t rank,
                        int64_t worldSize, int64_t dpSize, int64_t hiddenDim, int64_t hiddenDimBytes,
                        int64_t hiddenDimScaleBytes) {
  return create_rank("internode", "default", maxNumTokens, numExperts, expertsPerToken, rank, worldSize, dpSize,
                     hiddenDim, hiddenDimBytes, hiddenDimScaleBytes);
}

// ---------------------------------------------------------------------------
// Tensor checks (csrc/bindings/all_to_all_ops.cpp:19-24,135-161,249-259)
// ---------------------------------------------------------------------------
void check_tensor(const at::Tensor &x, int64_t ndim, const char *name) {
  TORCH_CHECK(x.is_cuda(), "Tensor ", name, " must be on GPU");
  TORCH_CHECK(x.is_contiguous(), "Tensor ", name, " must be contiguous");
  TORCH_CHECK(x.dim() == ndim, "Tensor ", name, " must be ", ndim, " dimensional");
}

void check_bound_m(const at::Tensor *bound_m) {
  if (!bound_m) return;
  check_tensor(*bound_m, 1, "boundM.value()");
  TORCH_CHECK(bound_m->scalar_type() == at::kUInt32, "boundM must be of type UInt32");
  TORCH_CHECK(bound_m->numel() == 1, "boundM must be a scalar tensor");
}

// getSplitMode, csrc/bindings/all_to_all_ops.cpp:110-120
int split_mode_of(bool do_send, bool do_recv) {
  TORCH_CHECK(do_send || do_recv, "Invalid split mode");
  if (do_send && do_recv) return PPLX_A2A_SPLIT_NONE;
  return do_send ? PPLX_A2A_SPLIT_SEND : PPLX_A2A_SPLIT_RECV;
}

int dtype_code(at::ScalarType t) {
  switch (t) {
    case at::kFloat: return PPLX_A2A_F32;
    case at::kBFloat16: return PPLX_A2A_BF16;
    case at::kHalf: return PPLX_A2A_F16;
    default: return -1;
  }
}

RankRef find_rank(fptr_t ptr) {
  auto it = g_ranks.find(ptr);
  TORCH_CHECK(it != g_ranks.end(), "pplx_kernels: invalid state: the handle has been destroyed");
  return it->second;
}

void reserve_split_locked(World &world, int expert_y_elem_bytes) {
  if (world.split_reserved >= expert_y_elem_bytes) return;
  A2A_CHECK(pplx_a2a_world_reserve_split(world.ptr, (uint32_t)expert_y_elem_bytes));
  world.split_reserved = expert_y_elem_bytes;
}

void clear_held(World &world, int op) {
  for (int mode = 0; mode < kModes; ++mode) {
    for (auto &tensors : world.held[op * kModes + mode]) tensors.clear();
  }
}

// After a call into the library: the tensors of a recorded call are kept, and everything kept
// for the phase is let go once the library holds no recorded call of it any more (the phase
// has been launched, or the library gave the step up).
void settle_held(World &world, uint32_t rank, int op, int mode, bool recorded,
                 std::initializer_list<const at::Tensor *> tensors) {
  uint32_t pending = 0;
  (void)pplx_a2a_world_recorded_calls(world.ptr, op, mode, &pending);
  auto &per_rank = world.held[op * kModes + mode];
  if (pending == 0) {
    for (auto &kept : per_rank) kept.clear();
    return;
  }
  if (!recorded) return;
  auto &kept = per_rank[rank];
  kept.clear();
  for (const at::Tensor *t : tensors) {
    if (t) kept.push_back(*t);
  }
}

// A rank whose arguments are refused after other ranks of the step have called would leave
// the world waiting for it for good (every retry of an earlier rank "called twice"): the step
// being assembled is given up, so that the caller can start it again from its first rank.
// Returns the number of recorded calls that were dropped.
uint32_t abandon_assembly(World *world, int op) {
  uint32_t dropped = 0;
  if (!world) return 0;
  (void)pplx_a2a_world_abandon_step(world->ptr, op == 0 ? PPLX_A2A_ABANDON_DISPATCH : PPLX_A2A_ABANDON_COMBINE,
                                    &dropped);
  clear_held(*world, op);
  return dropped;
}

#define A2A_RETHROW_ABANDONED(err, op_name, dropped)                                              \
  TORCH_CHECK(false, (err).what_without_backtrace(), " (the " op_name                             \
              " step that was being assembled has been abandoned: ", (dropped),                   \
              " recorded call(s) dropped, every rank calls again)")

void *current_stream_of(const at::Tensor &t) {
  return (void *)c10::hip::getCurrentHIPStream(t.device().index()).stream();
}

// csrc/bindings/all_to_all_ops.cpp:122-196.  Optional tensors arrive as pointers (NULL = None).
void dispatch_core(fptr_t ptr, const at::Tensor &outExpertNumTokens, const at::Tensor &outExpertX,
                   const at::Tensor *outExpertXScale, const at::Tensor &dpX, const at::Tensor *dpXScale,
                   const at::Tensor &indices, const at::Tensor *boundM, bool doSend, bool doRecv) {
  std::lock_guard<std::mutex> lock(g_mu);
  World *world = nullptr;
  // What a failure means: refused arguments give the step being assembled up (below); call-order
  // and runtime errors leave the recorded calls alone.
  bool arguments_refused = true;
  try {
    // (a handle that is unknown is reported after the tensor checks, which need no handle)
    auto found = g_ranks.find(ptr);
    if (found != g_ranks.end()) world = found->second.world;
    check_tensor(outExpertNumTokens, 1, "outExpertNumTokens");
    TORCH_CHECK(outExpertNumTokens.scalar_type() == at::kInt, "outExpertNumTokens must be of type Int");
    check_tensor(outExpertX, 3, "outExpertX");
    if (outExpertXScale) {
      TORCH_CHECK(outExpertXScale->is_cuda(), "Tensor outExpertXScale must be on GPU");
      TORCH_CHECK(outExpertXScale->dim() == 3, "Tensor outExpertXScale must be 3 dimensional");
      TORCH_CHECK(outExpertXScale->scalar_type() == at::kFloat, "outExpertXScale must be of type Float");
    }
    check_tensor(dpX, 2, "dpX");
    if (dpXScale) {
      TORCH_CHECK(dpXScale->is_cuda(), "Tensor dpXScale must be on GPU");
      TORCH_CHECK(dpXScale->dim() == 2, "Tensor dpXScale must be 2 dimensional");
      TORCH_CHECK(dpXScale->scalar_type() == at::kFloat, "dpXScale must be of type Float");
    }
    check_tensor(indices, 2, "indices");
    TORCH_CHECK(indices.scalar_type() == at::kUInt32, "indices must be of type UInt32");
    check_bound_m(boundM);
    TORCH_CHECK(indices.size(0) == dpX.size(0), "indices.size(0) must be equal to dpX.size(0)");
    const RankRef ref = find_rank(ptr);
    TORCH_CHECK(indices.size(1) == (int64_t)world->cfg.experts_per_token,
                "indices.size(1) must be equal to the experts per token");
    const int mode = split_mode_of(doSend, doRecv);

    pplx_a2a_dispatch_args_t a{};
    a.out_expert_num_tokens = static_cast<int32_t *>(outExpertNumTokens.data_ptr());
    a.out_expert_num_tokens_stride = outExpertNumTokens.stride(0);
    const int64_t esz = (int64_t)outExpertX.element_size();
    a.out_expert_x = outExpertX.data_ptr();
    a.out_expert_x_stride_row = outExpertX.stride(1) * esz;
    a.out_expert_x_stride_expert = outExpertX.stride(0) * esz;
    a.out_expert_x_rows = outExpertX.size(1);
    if (outExpertXScale) {
      a.out_expert_x_scale = static_cast<float *>(outExpertXScale->data_ptr());
      a.out_expert_x_scale_stride_elem = outExpertXScale->stride(2);
      a.out_expert_x_scale_stride_row = outExpertXScale->stride(1);
      a.out_expert_x_scale_stride_expert = outExpertXScale->stride(0);
    }
    a.dp_x = dpX.data_ptr();
    a.dp_x_stride_row = dpX.stride(0) * (int64_t)dpX.element_size();
    if (dpXScale) {
      a.dp_x_scale = static_cast<const float *>(dpXScale->data_ptr());
      a.dp_x_scale_stride_elem = dpXScale->stride(1);
      a.dp_x_scale_stride_row = dpXScale->stride(0);
    }
    a.indices = static_cast<const uint32_t *>(indices.data_ptr());
    a.m = (uint32_t)indices.size(0);
    a.bound_m = boundM ? static_cast<const uint32_t *>(boundM->data_ptr()) : nullptr;

    // Split calls go through staging that dispatch / combine never allocate; the reference's
    // callers do not know of it, so it is reserved the first time a rank splits a call.
    arguments_refused = false;
    if (mode != PPLX_A2A_SPLIT_NONE) reserve_split_locked(*world, 0);
    // The library selects the world's device for the launch and restores the caller's; the
    // stream is the current one of the tensors' device (csrc/bindings/all_to_all_ops.cpp:163,194).
    const int st = pplx_a2a_dispatch((pplx_a2a_t *)ptr, &a, mode, current_stream_of(indices));
    settle_held(*world, ref.rank, 0, mode, st == PPLX_A2A_OK,
                {&outExpertNumTokens, &outExpertX, outExpertXScale, &dpX, dpXScale, &indices, boundM});
    arguments_refused = st == PPLX_A2A_INVALID_ARGUMENT;
    A2A_CHECK(st);
  } catch (const c10::Error &err) {
    const uint32_t dropped = arguments_refused ? abandon_assembly(world, 0) : 0;
    if (dropped == 0) throw;
    A2A_RETHROW_ABANDONED(err, "dispatch", dropped);
  }
}

// csrc/bindings/all_to_all_ops.cpp:238-311
void combine_core(fptr_t ptr, const at::Tensor &outTokens, const at::Tensor &indices, const at::Tensor &weights,
                  const at::Tensor &expertY, const at::Tensor *boundM, bool doSend, bool doRecv) {
  std::lock_guard<std::mutex> lock(g_mu);
  World *world = nullptr;
  bool arguments_refused = true;
  try {
    auto found = g_ranks.find(ptr);
    if (found != g_ranks.end()) world = found->second.world;
    check_tensor(outTokens, 2, "outTokens");
    check_tensor(indices, 2, "indices");
    TORCH_CHECK(indices.scalar_type() == at::kUInt32, "indices must be of type UInt32");
    check_tensor(weights, 2, "weights");
    TORCH_CHECK(weights.scalar_type() == at::kFloat, "weights must be of type Float");
    check_tensor(expertY, 3, "expertY");
    check_bound_m(boundM);
    const int in_dtype = dtype_code(expertY.scalar_type());
    TORCH_CHECK(in_dtype >= 0, "Unsupported dtype for expertY");
    const int out_dtype = dtype_code(outTokens.scalar_type());
    TORCH_CHECK(out_dtype == PPLX_A2A_BF16 || out_dtype == PPLX_A2A_F16, "Unsupported dtype for outTokens");
    const RankRef ref = find_rank(ptr);
    const int mode = split_mode_of(doSend, doRecv);

    pplx_a2a_combine_args_t a{};
    a.out_tokens = outTokens.data_ptr();
    a.out_tokens_stride_row = outTokens.stride(0);
    a.out_dtype = out_dtype;
    a.indices = static_cast<const uint32_t *>(indices.data_ptr());
    a.weights = static_cast<const float *>(weights.data_ptr());
    a.weights_stride_row = weights.stride(0);
    a.expert_y = expertY.data_ptr();
    a.expert_y_stride_row = expertY.stride(1);
    a.expert_y_stride_expert = expertY.stride(0);
    a.expert_y_rows = expertY.size(1);
    a.in_dtype = in_dtype;
    a.m = (uint32_t)indices.size(0);
    a.bound_m = boundM ? static_cast<const uint32_t *>(boundM->data_ptr()) : nullptr;

    arguments_refused = false;
    if (mode != PPLX_A2A_SPLIT_NONE) reserve_split_locked(*world, (int)expertY.element_size());
    const int st = pplx_a2a_combine((pplx_a2a_t *)ptr, &a, mode, current_stream_of(indices));
    settle_held(*world, ref.rank, 1, mode, st == PPLX_A2A_OK, {&outTokens, &indices, &weights, &expertY, boundM});
    arguments_refused = st == PPLX_A2A_INVALID_ARGUMENT;
    A2A_CHECK(st);
  } catch (const c10::Error &err) {
    const uint32_t dropped = arguments_refused ? abandon_assembly(world, 1) : 0;
    if (dropped == 0) throw;
    A2A_RETHROW_ABANDONED(err, "combine", dropped);
  }
}

const at::Tensor *opt(const std::optional<at::Tensor> &t) { return t.has_value() ? &*t : nullptr; }

// The registered ops (the reference's signatures).
void dispatch_op(fptr_t ptr, at::Tensor &outExpertNumTokens, at::Tensor &outExpertX,
                 const std::optional<at::Tensor> &outExpertXScale, const at::Tensor &dpX,
                 const std::optional<at::Tensor> &dpXScale, const at::Tensor &indices,
                 const std::optional<at::Tensor> &boundM, bool doSend, bool doRecv) {
  dispatch_core(ptr, outExpertNumTokens, outExpertX, opt(outExpertXScale), dpX, opt(dpXScale), indices, opt(boundM),
                doSend, doRecv);
}

void combine_op(fptr_t ptr, at::Tensor &outTokens, const at::Tensor &indices, const at::Tensor &weights,
                const at::Tensor &expertY, const std::optional<at::Tensor> &boundM, bool doSend, bool doRecv) {
  combine_core(ptr, outTokens, indices, weights, expertY, opt(boundM), doSend, doRecv);
}

// Meta kernels: a traced call does nothing (csrc/bindings/all_to_all_ops.cpp:198-209,313-322).
void fake_dispatch(fptr_t, at::Tensor &, at::Tensor &, const std::optional<at::Tensor> &, const at::Tensor &,
                   const std::optional<at::Tensor> &, const at::Tensor &, const std::optional<at::Tensor> &, bool,
                   bool) {}

void fake_combine(fptr_t, at::Tensor &, const at::Tensor &, const at::Tensor &, const at::Tensor &,
                  const std::optional<at::Tensor> &, bool, bool) {}

const char *kDispatchArgs =
    "(int fptr, Tensor! out_expert_num_tokens, Tensor! out_expert_x, Tensor!? out_expert_x_scale, "
    "Tensor dp_x, Tensor? dp_x_scale, Tensor indices, Tensor? bound_m, bool do_send, bool do_recv) -> ()";
const char *kCombineArgs =
    "(int fptr, Tensor! out_tokens, Tensor indices, Tensor weights, Tensor expert_y, "
    "Tensor? bound_m, bool do_send, bool do_recv) -> ()";

}  // namespace

// csrc/bindings/bindings.cpp:9-12, csrc/bindings/all_to_all_ops.cpp:329-391
TORCH_LIBRARY(pplx_kernels, m) {
  m.def("all_to_all_destroy", &destroy);
  m.def("all_to_all_intranode_create", &create_intranode);
  m.def("all_to_all_internode_create", &create_internode);
  for (const char *transport : {"intranode", "internode"}) {
    const std::string dispatch = std::string("all_to_all_") + transport + "_dispatch";
    m.def((dispatch + kDispatchArgs).c_str());
    m.impl(dispatch.c_str(), c10::kCUDA, &dispatch_op);
    m.impl(dispatch.c_str(), c10::kMeta, &fake_dispatch);
    const std::string combine = std::string("all_to_all_") + transport + "_combine";
    m.def((combine + kCombineArgs).c_str());
    m.impl(combine.c_str(), c10::kCUDA, &combine_op);
    m.impl(combine.c_str(), c10::kMeta, &fake_combine);
  }
}

// ---------------------------------------------------------------------------
// Module pplx_kernels._C: the same entry points without the op dispatcher
// ---------------------------------------------------------------------------
namespace {

const at::Tensor &tensor_arg(PyObject *obj, const char *name) {
  TORCH_CHECK_TYPE(THPVariable_Check(obj), name, " must be a Tensor, not ", Py_TYPE(obj)->tp_name);
  return THPVariable_Unpack(obj);
}

const at::Tensor *optional_tensor_arg(PyObject *obj, const char *name) {
  return obj == Py_None ? nullptr : &tensor_arg(obj, name);
}

int64_t int_arg(PyObject *obj, const char *name) {
  const long long v = PyLong_AsLongLong(obj);
  if (v == -1 && PyErr_Occurred()) {
    PyErr_Clear();
    TORCH_CHECK_TYPE(false, name, " must be an int, not ", Py_TYPE(obj)->tp_name);
  }
  return v;
}

void arity(const char *fn, Py_ssize_t got, Py_ssize_t want) {
  TORCH_CHECK_TYPE(got == want, fn, "() takes ", want, " positional arguments but ", got, " were given");
}

// dispatch(fptr, out_expert_num_tokens, out_expert_x, out_expert_x_scale, dp_x, dp_x_scale, indices,
//          bound_m, do_send, do_recv)
PyObject *py_dispatch(PyObject *, PyObject *const *args, Py_ssize_t nargs) {
  HANDLE_TH_ERRORS
  arity("dispatch", nargs, 10);
  dispatch_core(int_arg(args[0], "fptr"), tensor_arg(args[1], "out_expert_num_tokens"),
                tensor_arg(args[2], "out_expert_x"), optional_tensor_arg(args[3], "out_expert_x_scale"),
                tensor_arg(args[4], "dp_x"), optional_tensor_arg(args[5], "dp_x_scale"),
                tensor_arg(args[6], "indices"), optional_tensor_arg(args[7], "bound_m"),
                PyObject_IsTrue(args[8]) == 1, PyObject_IsTrue(args[9]) == 1);
  Py_RETURN_NONE;
  END_HANDLE_TH_ERRORS
}

// combine(fptr, out_tokens, indices, weights, expert_y, bound_m, do_send, do_recv)
PyObject *py_combine(PyObject *, PyObject *const *args, Py_ssize_t nargs) {
  HANDLE_TH_ERRORS
  arity("combine", nargs, 8);
  combine_core(int_arg(args[0], "fptr"), tensor_arg(args[1], "out_tokens"), tensor_arg(args[2], "indices"),
               tensor_arg(args[3], "weights"), tensor_arg(args[4], "expert_y"),
               optional_tensor_arg(args[5], "bound_m"), PyObject_IsTrue(args[6]) == 1,
               PyObject_IsTrue(args[7]) == 1);
  Py_RETURN_NONE;
  END_HANDLE_TH_ERRORS
}

PyObject *py_destroy_all(PyObject *, PyObject *) {
  HANDLE_TH_ERRORS
  destroy_all();
  Py_RETURN_NONE;
  END_HANDLE_TH_ERRORS
}

PyObject *py_is_live(PyObject *, PyObject *arg) {
  HANDLE_TH_ERRORS
  const fptr_t ptr = int_arg(arg, "fptr");
  std::lock_guard<std::mutex> lock(g_mu);
  return PyBool_FromLong(g_ranks.count(ptr) != 0);
  END_HANDLE_TH_ERRORS
}

// world_ptr(fptr) -> the pplx_a2a_world_t * of the handle's world, as an int
PyObject *py_world_ptr(PyObject *, PyObject *arg) {
  HANDLE_TH_ERRORS
  const fptr_t ptr = int_arg(arg, "fptr");
  std::lock_guard<std::mutex> lock(g_mu);
  return PyLong_FromVoidPtr(find_rank(ptr).world->ptr);
  END_HANDLE_TH_ERRORS
}

// reserve_split(fptr, expert_y_elem_bytes)
PyObject *py_reserve_split(PyObject *, PyObject *const *args, Py_ssize_t nargs) {
  HANDLE_TH_ERRORS
  arity("reserve_split", nargs, 2);
  const fptr_t ptr = int_arg(args[0], "fptr");
  const int64_t bytes = int_arg(args[1], "expert_y_elem_bytes");
  std::lock_guard<std::mutex> lock(g_mu);
  reserve_split_locked(*find_rank(ptr).world, (int)bytes);
  Py_RETURN_NONE;
  END_HANDLE_TH_ERRORS
}

// abandon_step(fptr, which) -> recorded calls dropped; which: 1 dispatch, 2 combine, 3 both
PyObject *py_abandon_step(PyObject *, PyObject *const *args, Py_ssize_t nargs) {
  HANDLE_TH_ERRORS
  arity("abandon_step", nargs, 2);
  const fptr_t ptr = int_arg(args[0], "fptr");
  const int64_t which = int_arg(args[1], "which");
  std::lock_guard<std::mutex> lock(g_mu);
  World *world = find_rank(ptr).world;
  uint32_t dropped = 0;
  A2A_CHECK(pplx_a2a_world_abandon_step(world->ptr, (uint32_t)which, &dropped));
  if (which & PPLX_A2A_ABANDON_DISPATCH) clear_held(*world, 0);
  if (which & PPLX_A2A_ABANDON_COMBINE) clear_held(*world, 1);
  return PyLong_FromUnsignedLong(dropped);
  END_HANDLE_TH_ERRORS
}

// held_tensors(fptr) -> number of tensors the world keeps alive for recorded calls (for tests)
PyObject *py_held_tensors(PyObject *, PyObject *arg) {
  HANDLE_TH_ERRORS
  const fptr_t ptr = int_arg(arg, "fptr");
  std::lock_guard<std::mutex> lock(g_mu);
  size_t n = 0;
  for (const auto &per_rank : find_rank(ptr).world->held) {
    for (const auto &kept : per_rank) n += kept.size();
  }
  return PyLong_FromSize_t(n);
  END_HANDLE_TH_ERRORS
}

#ifndef PPLX_BINDING_SOURCE_ID
#define PPLX_BINDING_SOURCE_ID "unknown"
#endif
// build_id() -> hash of the sources this module was built from (a stale build shows up in a test)
PyObject *py_build_id(PyObject *, PyObject *) { return PyUnicode_FromString(PPLX_BINDING_SOURCE_ID); }

PyMethodDef kMethods[] = {
    {"build_id", py_build_id, METH_NOARGS, "hash of the sources the module was built from"},
    {"dispatch", (PyCFunction)(void (*)(void))py_dispatch, METH_FASTCALL,
     "dispatch(fptr, out_expert_num_tokens, out_expert_x, out_expert_x_scale, dp_x, dp_x_scale, indices, "
     "bound_m, do_send, do_recv): all_to_all_*_dispatch without the op dispatcher"},
    {"combine", (PyCFunction)(void (*)(void))py_combine, METH_FASTCALL,
     "combine(fptr, out_tokens, indices, weights, expert_y, bound_m, do_send, do_recv): all_to_all_*_combine "
     "without the op dispatcher"},
    {"destroy_all", py_destroy_all, METH_NOARGS, "releases every rank handle and world"},
    {"is_live", py_is_live, METH_O, "is_live(fptr) -> bool"},
    {"world_ptr", py_world_ptr, METH_O, "world_ptr(fptr) -> address of the handle's pplx_a2a_world_t"},
    {"reserve_split", (PyCFunction)(void (*)(void))py_reserve_split, METH_FASTCALL,
     "reserve_split(fptr, expert_y_elem_bytes)"},
    {"abandon_step", (PyCFunction)(void (*)(void))py_abandon_step, METH_FASTCALL,
     "abandon_step(fptr, which) -> recorded calls dropped"},
    {"held_tensors", py_held_tensors, METH_O, "held_tensors(fptr) -> tensors kept alive for recorded calls"},
    {nullptr, nullptr, 0, nullptr},
};

PyModuleDef kModule = {PyModuleDef_HEAD_INIT, "_C", "torch operator layer of pplx_kernels (see pplx_kernels.ops)",
                       -1, kMethods, nullptr, nullptr, nullptr, nullptr};

}  // namespace

PyMODINIT_FUNC PyInit__C(void) { return PyModule_Create(&kModule); }
