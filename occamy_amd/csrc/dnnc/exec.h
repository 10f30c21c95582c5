#pragma once
#include <map>
#include <string>
#include <vector>

#include "../../../include/dnnrt.h"
#include "ir.h"

namespace dnnc {

// The runtime's entry points, resolved by name from a shared object.
struct RuntimeApi {
  void *dl = nullptr;
  decltype(&::dnnrtCreate) dnnrtCreate = nullptr;
  decltype(&::dnnrtDestroy) dnnrtDestroy = nullptr;
  decltype(&::dnnrtDeviceMemoryStats) dnnrtDeviceMemoryStats = nullptr;
  decltype(&::dnnrtStreamCreate) dnnrtStreamCreate = nullptr;
  decltype(&::dnnrtStreamDestroy) dnnrtStreamDestroy = nullptr;
  decltype(&::dnnrtSetStream) dnnrtSetStream = nullptr;
  decltype(&::dnnrtSetTensorFormat) dnnrtSetTensorFormat = nullptr;
  decltype(&::dnnrtSetFilterLayout) dnnrtSetFilterLayout = nullptr;
  decltype(&::dnnrtSync) dnnrtSync = nullptr;
  decltype(&::dnnrtLastError) dnnrtLastError = nullptr;
  decltype(&::dnnrtIsHostBackend) dnnrtIsHostBackend = nullptr;
  decltype(&::dnnrtGraphBegin) dnnrtGraphBegin = nullptr;
  decltype(&::dnnrtGraphEnd) dnnrtGraphEnd = nullptr;
  decltype(&::dnnrtGraphLaunch) dnnrtGraphLaunch = nullptr;
  decltype(&::dnnrtGraphDestroy) dnnrtGraphDestroy = nullptr;
  decltype(&::dnnrtEventCreate) dnnrtEventCreate = nullptr;
  decltype(&::dnnrtEventRecord) dnnrtEventRecord = nullptr;
  decltype(&::dnnrtEventElapsedMs) dnnrtEventElapsedMs = nullptr;
  decltype(&::dnnrtEventDestroy) dnnrtEventDestroy = nullptr;
  decltype(&::dnnrtMemPoolInit) dnnrtMemPoolInit = nullptr;
  decltype(&::dnnrtMemOffset) dnnrtMemOffset = nullptr;
  decltype(&::dnnrtMemcpy) dnnrtMemcpy = nullptr;
  decltype(&::dnnrtMalloc) dnnrtMalloc = nullptr;
  decltype(&::dnnrtDealloc) dnnrtDealloc = nullptr;
  decltype(&::dnnrtHostAlloc) dnnrtHostAlloc = nullptr;
  decltype(&::dnnrtHostFree) dnnrtHostFree = nullptr;
  decltype(&::dnnrtConv) dnnrtConv = nullptr;
  decltype(&::dnnrtConvBiasActiv) dnnrtConvBiasActiv = nullptr;
  decltype(&::dnnrtConvBiasAddActiv) dnnrtConvBiasAddActiv = nullptr;
  decltype(&::dnnrtConvBiasActivMaxPool) dnnrtConvBiasActivMaxPool = nullptr;
  decltype(&::dnnrtConvBiasAddConvBiasActiv) dnnrtConvBiasAddConvBiasActiv = nullptr;
  decltype(&::dnnrtActive) dnnrtActive = nullptr;
  decltype(&::dnnrtTensorOp) dnnrtTensorOp = nullptr;
  decltype(&::dnnrtClip) dnnrtClip = nullptr;
  decltype(&::dnnrtErf) dnnrtErf = nullptr;
  decltype(&::dnnrtNegative) dnnrtNegative = nullptr;
  decltype(&::dnnrtReciprocal) dnnrtReciprocal = nullptr;
  decltype(&::dnnrtPow) dnnrtPow = nullptr;
  decltype(&::dnnrtCastI64toFloat) dnnrtCastI64toFloat = nullptr;
  decltype(&::dnnrtGelu) dnnrtGelu = nullptr;
  decltype(&::dnnrtReduce) dnnrtReduce = nullptr;
  decltype(&::dnnrtSoftmax) dnnrtSoftmax = nullptr;
  decltype(&::dnnrtLayerNorm) dnnrtLayerNorm = nullptr;
  decltype(&::dnnrtMaxPool) dnnrtMaxPool = nullptr;
  decltype(&::dnnrtAveragePool) dnnrtAveragePool = nullptr;
  decltype(&::dnnrtMatmul2d) dnnrtMatmul2d = nullptr;
  decltype(&::dnnrtMatmulNd) dnnrtMatmulNd = nullptr;
  decltype(&::dnnrtFlatten) dnnrtFlatten = nullptr;
  decltype(&::dnnrtReshape) dnnrtReshape = nullptr;
  decltype(&::dnnrtTranspose) dnnrtTranspose = nullptr;
  decltype(&::dnnrtGather) dnnrtGather = nullptr;
  decltype(&::dnnrtSetActivationCoef) dnnrtSetActivationCoef = nullptr;
  decltype(&::dnnrtSetConvTile) dnnrtSetConvTile = nullptr;
  decltype(&::dnnrtListConvTiles) dnnrtListConvTiles = nullptr;
  decltype(&::dnnrtMemFill) dnnrtMemFill = nullptr;
  decltype(&::dnnrtMatmulNdBias) dnnrtMatmulNdBias = nullptr;
  decltype(&::dnnrtAttention) dnnrtAttention = nullptr;
  decltype(&::dnnrtLeakyRelu) dnnrtLeakyRelu = nullptr;
  decltype(&::dnnrtPRelu) dnnrtPRelu = nullptr;
  decltype(&::dnnrtConcat) dnnrtConcat = nullptr;
  decltype(&::dnnrtSqueeze) dnnrtSqueeze = nullptr;
  decltype(&::dnnrtUnsqueeze) dnnrtUnsqueeze = nullptr;
  decltype(&::dnnrtExpand) dnnrtExpand = nullptr;
};

bool load_runtime(const std::string &path, RuntimeApi &rt, std::string &err);

enum { MODE_OCCAMY = 0, MODE_RESIDENT = 1 };

class Session {
 public:
  ~Session();
  bool init(const Program *p, const std::string &runtime_path, int mode, std::string &err);
  bool run_occamy(const void *const *inputs, void *const *outputs, std::string &err);
  bool run_resident(const void *const *inputs, void *const *outputs, int on_device, int use_graph, std::string &err);
  bool sync(std::string &err);
  // Tuning: dnnrtSetConvTile on the session's handle; a captured graph is dropped (it holds the old variants).
  bool set_conv_tile(int tile, std::string &err);
  // Resident mode: one eager pass with a device timestamp around every compute
  // operation; ms[i] is the time of the i-th compute op in program order.
  // by_class: timestamps only around each operation class's launches issued
  // back to back; ms[i] is then the class average.
  bool profile_resident(const void *const *inputs, int on_device, bool by_class, std::vector<float> &ms, std::string &err);
  bool profile_classes(const void *const *inputs, int on_device, const std::vector<const Op *> &compute,
                       std::vector<float> &ms, std::string &err);

  // The measured choice of convolution variant, where the reference times cuDNN's algorithms at compile time
  // and passes the winner as the call's `algo` operand (src/Conversion/ONNXToDNN/ONNXToDNNCommonCUDA.cu:57-111).
  // Resident sessions on the GPU runtime: every variant the runtime lists is tried on every convolution of the
  // program in place, i.e. timed inside whole passes over the program (a layer's operands are then where the
  // layers before it leave them: in HBM or in a cache); a variant replaces the runtime's own choice for an
  // operation when it is faster by more than 3 % in the median of `reps` passes.  `changed`: how many operations
  // got a variant.  A session on the host build of the ABI, or a program without fp16 channels-last convolutions,
  // has nothing to tune (changed = 0).
  bool tune(const void *const *inputs, int on_device, int reps, int64_t &changed, std::string &err);
  // The choices, two per operation that launches (dnncProgramComputeOp order): the `algo` operand and, for a
  // fused shortcut pair, that of its second convolution; 0 = the runtime's own choice.
  std::vector<int64_t> algos() const;
  bool set_algos(const int64_t *a, int64_t n, std::string &err);

  const Program *prog = nullptr;
  int mode = MODE_OCCAMY;
  int64_t weights_bytes = 0;     // bytes of the constants arena (resident mode)
  // Debugging (the reference's per-inference mode): fill the pool when it is allocated and every tensor's slot when
  // it is carved out with this byte (-1: off); 0xFF makes any byte a kernel leaves unwritten, or reads before its
  // producer ran, a NaN in the results.
  int debug_fill = -1;
  int64_t last_pool_bytes = -1;  // bytes the last occamy-mode run asked the runtime for
  // the bound runtime library's device-memory accounting (dnnrtDeviceMemoryStats)
  int device_bytes(int64_t *now, int64_t *peak, int64_t *static_bytes, int reset_peak) const {
    return rt.dnnrtDeviceMemoryStats ? rt.dnnrtDeviceMemoryStats(now, peak, static_bytes, reset_peak) : 1;
  }

 private:
  RuntimeApi rt;
  dnnrtHandle_t handle = nullptr;
  dnnrtStream_t stream = nullptr;
  bool host_backend = false;
  int cur_format = 0, cur_filter_layout = 0;
  float cur_act_coef = 0.f;   // what the handle's activation coefficient was last set to
  std::map<std::string, bool> crsk_const;  // constants re-laid C,R,S,K on the host
  std::vector<char> filter_crsk;           // value id -> its device copy is C,R,S,K
  void *pool = nullptr, *weights = nullptr, *graph = nullptr;
  // Recorded graphs of other argument / result addresses than the current ones (runs in place hold the caller's
  // addresses in the graph): a caller that alternates between a few sets of buffers gets its graph back instead
  // of a new recording each time.  At most four; the oldest goes first.
  std::vector<std::pair<std::vector<void *>, void *>> parked_graphs;
  std::vector<void *> graph_key;  // the addresses `graph` was recorded with
  void drop_graphs();
  std::vector<void *> ptr;  // value id -> address (host or device)
  std::map<const Op *, std::pair<int64_t, int64_t>> tuned;  // operation -> variant ids of its one or two convolutions (0: automatic)
  int64_t algo_operand(const Op *op, int which, int64_t reference_value) const;
  std::map<size_t, void *> arg_home;  // resident mode: value id of a function argument's pool slot -> its address in the pool
  std::vector<const Op *> direct_out;  // the result copies of the current run that are not needed for that reason
  std::map<size_t, void *> out_home;  // ... and of a result's pool tensor, when results are written where the caller wants them
  std::map<std::string, void *> host_const;
  std::vector<void *> host_out, host_in;
  // resident mode: results produced mid-program, whose pool bytes a later
  // tensor may take over, are copied aside (on the device, in program order)
  std::map<const Op *, void *> staged_out;  // the device-to-host memcpy op -> its staging buffer

  std::string rt_error(const char *what) const;
  int format_for(const Op *op) const;
  bool issue(const Op *op, std::string &err);
  bool issue_all_compute(std::string &err);
};

}  // namespace dnnc
