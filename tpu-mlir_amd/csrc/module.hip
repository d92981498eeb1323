// Device-resident mini-interpreter: a list of the ops this library implements, run back to back on one stream with
// every activation staying in HBM in its native storage type.  It is the shape of the reference's GPU interpreter
// (bindings/pymlir/pycuda.cpp: gpu_load :17-49 uploads native-dtype weights once, set_tensor :399-436 converts the
// float input on the device, gpu_invoke :438-669 walks the ops, cuda_to_host/get_tensor :289-397,954-966 expand the
// result to float), without the MLIR parsing in front of it: the caller adds tensors and ops programmatically.
#include <algorithm>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "internal.h"

namespace {

using namespace mi;

int st_bytes(int t) {
  return (t == MI_ST_F32 || t == MI_ST_I32 || t == MI_ST_U32) ? 4 : ((t == MI_ST_I8 || t == MI_ST_U8) ? 1 : 2);
}

struct DevMem {
  void *ptr = nullptr;
  int alloc(size_t bytes) {
    MI_HIP(hipMalloc(&ptr, bytes ? bytes : 4));
    return MI_SUCCESS;
  }
  ~DevMem() {
    if (ptr)
      (void)hipFree(ptr);
  }
  DevMem() = default;
  DevMem(const DevMem &) = delete;
  DevMem &operator=(const DevMem &) = delete;
};

struct Tensor {
  std::string name;
  int st = MI_ST_F32;
  int64_t n = 0;
  std::unique_ptr<DevMem> mem;  // its own allocation, or empty once the tensor lives in the module's arena
  void *planned = nullptr;      // address inside the arena (mi_module_plan_memory)
  bool is_output = false;       // kept readable after invoke whatever the memory plan does
  bool shares_memory = false;   // its arena bytes are reused by other tensors: contents are gone after invoke
  bool quant = false;           // uniform-quantized: get_tensor scales it back (pycuda.cpp:326-343, :370-379)
  double q_scale = 1.0;
  int64_t q_zp = 0;
  void *ptr() const { return planned ? planned : mem->ptr; }
};

enum OpKind { OP_A16, OP_I8, OP_CAST, OP_REQUANT, OP_MATMUL_DQ };

struct Op {
  OpKind kind;
  int in = -1, out = -1;
  // A16MatMul
  mi_a16_weight *w = nullptr;
  int64_t M = 0;
  int dq_type = MI_DQ_NONE;  // dynamic activation quantization of this A16MatMul
  // quantized MatMul
  std::unique_ptr<DevMem> right, bias, mult, shift, zp;
  int64_t K = 0, N = 0;
  int a_unsigned = 0, b_unsigned = 0;
  int64_t input_zp = 0, right_zp = 0;
  int do_relu = 0;
  int64_t relu_limit = -1;
  bool has_rq = false;
  mi_requant_desc rq{};
  // Cast
  mi_cast_attr cast{};
  float inv_scale = 1.0f, scale = 1.0f;
  // standalone requant
  int64_t outer = 1, channels = 1, inner = 1;
  // MatMul of two activations with dynamic quantization of both
  int in2 = -1, right_transpose = 0, q_group_size = 0, dtype = MI_DT_BF16;
  bool capturable = true;
};

}  // namespace

struct mi_module {
  std::vector<Tensor> tensors;
  std::map<std::string, int> index;
  std::vector<Op> ops;
  hipStream_t stream = nullptr;
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  bool graph_tried = false;
  DevMem staging;  // float staging for set_tensor / get_tensor
  size_t staging_bytes = 0;
  std::unique_ptr<DevMem> arena;  // one allocation shared by the activations whose lifetimes do not overlap
  mi_module_hook before = nullptr, after = nullptr;
  void *hook_user = nullptr;
  ~mi_module() {
    if (exec)
      (void)hipGraphExecDestroy(exec);
    if (graph)
      (void)hipGraphDestroy(graph);
    for (auto &o : ops)
      if (o.w)
        mi_a16_weight_destroy(o.w);
    if (stream) {
      mi::release_stream_workspaces(stream);  // after the graph that may name them
      (void)hipStreamDestroy(stream);
    }
  }
};

namespace {

int find(mi_module *m, const char *name, int *idx) {
  MI_REQUIRE(m && name, MI_BAD_ARGUMENT, "mi_module: null argument");
  auto it = m->index.find(name);
  MI_REQUIRE(it != m->index.end(), MI_BAD_ARGUMENT, std::string("mi_module: no tensor named '") + name + "'");
  *idx = it->second;
  return MI_SUCCESS;
}

int upload(std::unique_ptr<DevMem> &dst, const void *src, size_t bytes) {
  dst.reset(new DevMem());
  int rc = dst->alloc(bytes);
  if (rc)
    return rc;
  MI_HIP(hipMemcpy(dst->ptr, src, bytes, hipMemcpyHostToDevice));
  return MI_SUCCESS;
}

int need_staging(mi_module *m, size_t bytes) {
  if (bytes <= m->staging_bytes)
    return MI_SUCCESS;
  if (m->staging.ptr)
    (void)hipFree(m->staging.ptr);
  m->staging.ptr = nullptr;
  m->staging_bytes = 0;
  int rc = m->staging.alloc(bytes);
  if (rc)
    return rc;
  m->staging_bytes = bytes;
  return MI_SUCCESS;
}

void drop_graph(mi_module *m) {
  if (m->exec)
    (void)hipGraphExecDestroy(m->exec);
  if (m->graph)
    (void)hipGraphDestroy(m->graph);
  m->exec = nullptr;
  m->graph = nullptr;
  m->graph_tried = false;
}

// plain storage conversion (the interpreter's float view <-> native storage): a Cast with no quantization on either
// side; values are already representable in the target type, so nothing is rounded or clamped
mi_cast_attr plain_cast(int in_t, int out_t, int64_t n) {
  mi_cast_attr c{};
  c.num_elem = n;
  c.in_type = in_t;
  c.out_type = out_t;
  c.scale = 1.0;
  c.expressed = MI_ST_F32;
  c.round_mode = MI_ROUND_HALF_AWAY_FROM_ZERO;
  c.chip = MI_CHIP_BM168X;
  return c;
}

// The launches an op list turns into: consecutive A16MatMuls that read the same tensor with compatible weight sets
// (the q/k/v and gate/up siblings) go out as one grouped launch.  Returns how many ops the launch starting at op i
// covers, never reaching past `end`.
size_t launch_len(const mi_module *m, size_t i, size_t end) {
  const Op &o = m->ops[i];
  if (o.kind != OP_A16 || o.dq_type != MI_DQ_NONE)
    return 1;
  size_t g = 1;
  while (g < 4 && i + g < end) {
    const Op &c = m->ops[i + g];
    if (c.kind != OP_A16 || c.dq_type != MI_DQ_NONE || c.in != o.in || c.M != o.M || c.w->K != o.w->K || c.w->bits != o.w->bits ||
        c.w->g != o.w->g || c.w->dtype != o.w->dtype || c.w->chip != o.w->chip)
      break;
    ++g;
  }
  return g;
}

// Enqueues the ops [first, end) on the module's stream.  With hooks, each launch is bracketed by the before hook of
// its ops and -- after the stream has drained, so that the hook may read tensors -- their after hook, as
// ModuleInterpreter::invoke_all_in_mem brackets every op (host/ModuleInterpreter.cpp:637-989 with :1531-1540).
int enqueue_range(mi_module *m, size_t first, size_t end, bool with_hooks) {
  for (size_t i = first; i < end;) {
    Op &o = m->ops[i];
    Tensor &tin = m->tensors[o.in], &tout = m->tensors[o.out];
    int rc = MI_SUCCESS;
    const size_t step = launch_len(m, i, end);
    if (with_hooks && m->before)
      for (size_t k = 0; k < step; ++k)
        m->before(m->tensors[m->ops[i + k].out].name.c_str(), m->hook_user);
    switch (o.kind) {
    case OP_A16: {
      if (o.dq_type != MI_DQ_NONE) {  // dynamic activation quantization: its own pair of kernels, one op per launch
        rc = a16_dq_launch(o.w, o.dq_type, (const uint16_t *)tin.ptr(), o.M, (uint16_t *)tout.ptr(), nullptr,
                           m->stream);
        break;
      }
      const mi_a16_weight *ws[4];
      uint16_t *ys[4];
      for (size_t k = 0; k < step; ++k) {
        ws[k] = m->ops[i + k].w;
        ys[k] = (uint16_t *)m->tensors[m->ops[i + k].out].ptr();
      }
      rc = a16_launch_group(ws, (int)step, (const uint16_t *)tin.ptr(), o.M, ys, nullptr, m->stream);
      break;
    }
    case OP_I8:
      rc = i8mm_launch(tin.ptr(), o.a_unsigned, o.right->ptr, o.b_unsigned, /*right_transpose=*/1,
                       o.bias ? (const int32_t *)o.bias->ptr : nullptr, o.M, o.K, o.N, o.input_zp, o.right_zp,
                       o.do_relu, o.relu_limit, o.has_rq ? &o.rq : nullptr, tout.ptr(), nullptr, m->stream);
      break;
    case OP_CAST:
      rc = cast_launch(&o.cast, tin.ptr(), tout.ptr(), o.cast.num_elem, o.inv_scale, o.scale, false, m->stream);
      break;
    case OP_REQUANT:
      rc = requant_launch((const int32_t *)tin.ptr(), tout.ptr(), o.outer, o.channels, o.inner, o.input_zp,
                          &o.rq, m->stream);
      break;
    case OP_MATMUL_DQ:
      rc = matmul_dq_launch((const uint16_t *)tin.ptr(), (const uint16_t *)m->tensors[o.in2].ptr(),
                            o.right_transpose, o.M, o.K, o.N, o.q_group_size, o.dq_type, o.dtype,
                            (uint16_t *)tout.ptr(), nullptr, m->stream);
      break;
    }
    if (rc)
      return rc;
    if (with_hooks && m->after) {
      MI_HIP(hipStreamSynchronize(m->stream));
      for (size_t k = 0; k < step; ++k)
        m->after(m->tensors[m->ops[i + k].out].name.c_str(), m->hook_user);
    }
    i += step;
  }
  return MI_SUCCESS;
}

int enqueue_all(mi_module *m) { return enqueue_range(m, 0, m->ops.size(), false); }

// the op that writes tensor `name` (ops are named after their output, as the reference names them)
int find_op(mi_module *m, const char *name, size_t *op) {
  int idx, rc;
  if ((rc = find(m, name, &idx)))
    return rc;
  for (size_t i = 0; i < m->ops.size(); ++i)
    if (m->ops[i].out == idx) {
      *op = i;
      return MI_SUCCESS;
    }
  set_error(std::string("mi_module: no op writes '") + name + "'");
  return MI_BAD_ARGUMENT;
}

}  // namespace

extern "C" {

int mi_module_create(mi_module **out) {
  MI_REQUIRE(out, MI_BAD_ARGUMENT, "mi_module_create: null argument");
  MI_REQUIRE(mi_device_count() > 0, MI_HIP_ERROR, "mi_module_create: no GPU visible");
  std::unique_ptr<mi_module> m(new mi_module());
  MI_HIP(hipStreamCreate(&m->stream));
  *out = m.release();
  return MI_SUCCESS;
}

void mi_module_destroy(mi_module *m) { delete m; }

int mi_module_add_tensor(mi_module *m, const char *name, int storage_type, int64_t num_elem) {
  MI_REQUIRE(!m || !m->arena, MI_BAD_ARGUMENT, "mi_module: the memory plan is made; tensors and ops can no longer be added");
  MI_REQUIRE(m && name, MI_BAD_ARGUMENT, "mi_module_add_tensor: null argument");
  MI_REQUIRE(storage_type >= MI_ST_F32 && storage_type <= MI_ST_U32 && num_elem > 0, MI_BAD_ARGUMENT,
             "mi_module_add_tensor: bad storage type or size");
  MI_REQUIRE(!m->index.count(name), MI_BAD_ARGUMENT, std::string("mi_module_add_tensor: duplicate tensor '") + name + "'");
  Tensor t;
  t.name = name;
  t.st = storage_type;
  t.n = num_elem;
  t.mem.reset(new DevMem());
  int rc = t.mem->alloc((size_t)num_elem * st_bytes(storage_type));
  if (rc)
    return rc;
  m->index[name] = (int)m->tensors.size();
  m->tensors.push_back(std::move(t));
  return MI_SUCCESS;
}

int mi_module_add_a16matmul(mi_module *m, const char *input, const char *output, const mi_a16_weight_desc *desc,
                            const void *weight, const uint16_t *scale, const uint8_t *zp, const float *bias) {
  return mi_module_add_a16matmul_dq(m, input, output, desc, MI_DQ_NONE, weight, scale, zp, bias);
}

int mi_module_add_a16matmul_dq(mi_module *m, const char *input, const char *output, const mi_a16_weight_desc *desc,
                               int dq_type, const void *weight, const uint16_t *scale, const uint8_t *zp,
                               const float *bias) {
  MI_REQUIRE(!m || !m->arena, MI_BAD_ARGUMENT, "mi_module: the memory plan is made; tensors and ops can no longer be added");
  int in, out, rc;
  MI_REQUIRE(dq_type == MI_DQ_NONE || dq_type == MI_DQ_INT || dq_type == MI_DQ_F8E4M3 || dq_type == MI_DQ_F4,
             MI_UNSUPPORTED, "mi_module_add_a16matmul_dq: dq_type must be MI_DQ_NONE, MI_DQ_INT, MI_DQ_F8E4M3 or MI_DQ_F4");
  if ((rc = find(m, input, &in)) || (rc = find(m, output, &out)))
    return rc;
  MI_REQUIRE(desc, MI_BAD_ARGUMENT, "mi_module_add_a16matmul: null descriptor");
  MI_REQUIRE(in != out, MI_BAD_ARGUMENT, "mi_module_add_a16matmul: a matmul cannot write the tensor it reads");
  const int st = desc->dtype == MI_DT_F16 ? MI_ST_F16 : MI_ST_BF16;
  const Tensor &ti = m->tensors[in], &to = m->tensors[out];
  MI_REQUIRE(ti.st == st && to.st == st, MI_BAD_ARGUMENT,
             "mi_module_add_a16matmul: input and output must be stored in the weight set's 16-bit type");
  MI_REQUIRE(desc->K > 0 && ti.n % desc->K == 0, MI_BAD_ARGUMENT, "mi_module_add_a16matmul: input size is not M * K");
  const int64_t M = ti.n / desc->K;
  MI_REQUIRE(to.n == M * desc->N, MI_BAD_ARGUMENT, "mi_module_add_a16matmul: output size is not M * N");
  Op o;
  o.kind = OP_A16;
  o.in = in;
  o.out = out;
  o.M = M;
  o.dq_type = dq_type;
  rc = mi_a16_weight_create(&o.w, desc, weight, scale, zp, bias);
  if (rc)
    return rc;
  if (dq_type != MI_DQ_NONE) {
    // the shapes and code types the dynamic kernels handle are checked now, not at the first invoke: a launch with
    // no rows runs every check and nothing else
    rc = a16_dq_launch(o.w, dq_type, nullptr, 0, nullptr, nullptr, m->stream);
    if (rc) {
      mi_a16_weight_destroy(o.w);
      return rc;
    }
  }
  m->ops.push_back(std::move(o));
  drop_graph(m);
  return MI_SUCCESS;
}

int mi_module_add_matmul_int8(mi_module *m, const char *input, const char *output, const mi_module_i8_desc *d) {
  MI_REQUIRE(!m || !m->arena, MI_BAD_ARGUMENT, "mi_module: the memory plan is made; tensors and ops can no longer be added");
  int in, out, rc;
  if ((rc = find(m, input, &in)) || (rc = find(m, output, &out)))
    return rc;
  MI_REQUIRE(d && d->right, MI_BAD_ARGUMENT, "mi_module_add_matmul_int8: null descriptor or weight");
  MI_REQUIRE(in != out, MI_BAD_ARGUMENT, "mi_module_add_matmul_int8: a matmul cannot write the tensor it reads");
  const Tensor &ti = m->tensors[in], &to = m->tensors[out];
  MI_REQUIRE(ti.st == MI_ST_I8 || ti.st == MI_ST_U8, MI_BAD_ARGUMENT, "mi_module_add_matmul_int8: input must be 8-bit");
  MI_REQUIRE(d->K > 0 && d->N > 0 && ti.n % d->K == 0, MI_BAD_ARGUMENT, "mi_module_add_matmul_int8: input size is not M * K");
  const int64_t M = ti.n / d->K;
  MI_REQUIRE(to.n == M * d->N, MI_BAD_ARGUMENT, "mi_module_add_matmul_int8: output size is not M * N");
  Op o;
  o.kind = OP_I8;
  o.in = in;
  o.out = out;
  o.M = M;
  o.K = d->K;
  o.N = d->N;
  o.a_unsigned = ti.st == MI_ST_U8;
  o.b_unsigned = d->right_unsigned;
  o.input_zp = d->input_zp;
  o.right_zp = d->right_zp;
  o.do_relu = d->do_relu;
  o.relu_limit = d->relu_limit;
  // the weight is kept [N, K] (transposed once here when it comes as [K, N])
  std::vector<uint8_t> nk;
  const uint8_t *src = (const uint8_t *)d->right;
  if (!d->right_transpose) {
    nk.resize((size_t)d->K * d->N);
    for (int64_t k = 0; k < d->K; ++k)
      for (int64_t n = 0; n < d->N; ++n)
        nk[(size_t)n * d->K + k] = src[(size_t)k * d->N + n];
    src = nk.data();
  }
  if ((rc = upload(o.right, src, (size_t)d->K * d->N)))
    return rc;
  if (d->bias && (rc = upload(o.bias, d->bias, (size_t)d->N * 4)))
    return rc;
  o.has_rq = d->has_requant != 0;
  if (o.has_rq) {
    o.rq = d->rq;
    const int want = o.rq.out_dtype == MI_DT_I8 ? MI_ST_I8 : o.rq.out_dtype == MI_DT_U8 ? MI_ST_U8
                   : o.rq.out_dtype == MI_DT_I16 ? MI_ST_I16 : o.rq.out_dtype == MI_DT_U16 ? MI_ST_U16 : MI_ST_I32;
    MI_REQUIRE(to.st == want, MI_BAD_ARGUMENT, "mi_module_add_matmul_int8: output storage differs from the requant type");
    // per-channel arrays arrive as HOST pointers in this descriptor and move to the device here; being host arrays
    // they can be range-checked for the 32-bit epilogue on the spot
    o.rq.per_channel_q31_checked = 1;
    for (int64_t n = 0; n < d->N; ++n) {
      if (d->rq.d_shift && (d->rq.d_shift[n] < 1 || d->rq.d_shift[n] > 31))
        o.rq.per_channel_q31_checked = 0;
      if (d->rq.d_multiplier && d->rq.d_multiplier[n] == INT32_MIN)
        o.rq.per_channel_q31_checked = 0;
    }
    if (d->rq.d_multiplier) {
      if ((rc = upload(o.mult, d->rq.d_multiplier, (size_t)d->N * 4)))
        return rc;
      o.rq.d_multiplier = (const int32_t *)o.mult->ptr;
    }
    if (d->rq.d_shift) {
      if ((rc = upload(o.shift, d->rq.d_shift, (size_t)d->N * 4)))
        return rc;
      o.rq.d_shift = (const int32_t *)o.shift->ptr;
    }
    if (d->rq.d_zp) {
      if ((rc = upload(o.zp, d->rq.d_zp, (size_t)d->N * 4)))
        return rc;
      o.rq.d_zp = (const int32_t *)o.zp->ptr;
    }
  } else {
    MI_REQUIRE(to.st == MI_ST_I32, MI_BAD_ARGUMENT, "mi_module_add_matmul_int8: an un-requantized output is int32");
  }
  // zero points and unsigned operands make the launch allocate scratch: such ops stay out of a captured graph
  o.capturable = !o.a_unsigned && !o.b_unsigned && o.input_zp == 0 && o.right_zp == 0;
  m->ops.push_back(std::move(o));
  drop_graph(m);
  return MI_SUCCESS;
}

int mi_module_add_requant(mi_module *m, const char *input, const char *output, const mi_module_rq_desc *d) {
  MI_REQUIRE(!m || !m->arena, MI_BAD_ARGUMENT, "mi_module: the memory plan is made; tensors and ops can no longer be added");
  int in, out, rc;
  if ((rc = find(m, input, &in)) || (rc = find(m, output, &out)))
    return rc;
  MI_REQUIRE(d, MI_BAD_ARGUMENT, "mi_module_add_requant: null descriptor");
  const Tensor &ti = m->tensors[in], &to = m->tensors[out];
  MI_REQUIRE(ti.st == MI_ST_I32, MI_BAD_ARGUMENT, "mi_module_add_requant: the input must be an int32 tensor");
  MI_REQUIRE(d->outer > 0 && d->channels > 0 && d->inner > 0 && ti.n == d->outer * d->channels * d->inner && to.n == ti.n,
             MI_BAD_ARGUMENT, "mi_module_add_requant: tensor sizes are not outer * channels * inner");
  const int want = d->rq.out_dtype == MI_DT_I8 ? MI_ST_I8 : d->rq.out_dtype == MI_DT_U8 ? MI_ST_U8
                 : d->rq.out_dtype == MI_DT_I16 ? MI_ST_I16 : d->rq.out_dtype == MI_DT_U16 ? MI_ST_U16 : -1;
  MI_REQUIRE(want >= 0 && to.st == want, MI_BAD_ARGUMENT,
             "mi_module_add_requant: output storage differs from the requant type");
  Op o;
  o.kind = OP_REQUANT;
  o.in = in;
  o.out = out;
  o.outer = d->outer;
  o.channels = d->channels;
  o.inner = d->inner;
  o.input_zp = d->input_zp;
  o.rq = d->rq;
  // per-channel arrays arrive as HOST pointers in this descriptor and move to the device here
  if (d->rq.d_multiplier) {
    if ((rc = upload(o.mult, d->rq.d_multiplier, (size_t)d->channels * 4)))
      return rc;
    o.rq.d_multiplier = (const int32_t *)o.mult->ptr;
  }
  if (d->rq.d_shift) {
    if ((rc = upload(o.shift, d->rq.d_shift, (size_t)d->channels * 4)))
      return rc;
    o.rq.d_shift = (const int32_t *)o.shift->ptr;
  }
  if (d->rq.d_zp) {
    if ((rc = upload(o.zp, d->rq.d_zp, (size_t)d->channels * 4)))
      return rc;
    o.rq.d_zp = (const int32_t *)o.zp->ptr;
  }
  // modes, rounding and chip are checked by the launch itself: a launch over no elements validates them here
  rc = requant_launch((const int32_t *)ti.ptr(), to.ptr(), 0, d->channels, d->inner, d->input_zp, &o.rq, m->stream);
  if (rc)
    return rc;
  m->ops.push_back(std::move(o));
  drop_graph(m);
  return MI_SUCCESS;
}

int mi_module_add_matmul_dq(mi_module *m, const char *left, const char *right, const char *output, int64_t K,
                            int64_t N, int right_transpose, int q_group_size, int dq_type) {
  MI_REQUIRE(!m || !m->arena, MI_BAD_ARGUMENT, "mi_module: the memory plan is made; tensors and ops can no longer be added");
  int in, in2, out, rc;
  if ((rc = find(m, left, &in)) || (rc = find(m, right, &in2)) || (rc = find(m, output, &out)))
    return rc;
  const Tensor &tl = m->tensors[in], &tr = m->tensors[in2], &to = m->tensors[out];
  MI_REQUIRE(out != in && out != in2, MI_BAD_ARGUMENT, "mi_module_add_matmul_dq: a matmul cannot write a tensor it reads");
  MI_REQUIRE((tl.st == MI_ST_BF16 || tl.st == MI_ST_F16) && tr.st == tl.st && to.st == tl.st, MI_BAD_ARGUMENT,
             "mi_module_add_matmul_dq: the three tensors must share one 16-bit float type");
  MI_REQUIRE(K > 0 && N > 0 && tl.n % K == 0 && tr.n == K * N && to.n == tl.n / K * N, MI_BAD_ARGUMENT,
             "mi_module_add_matmul_dq: tensor sizes are not M * K, K * N and M * N");
  Op o;
  o.kind = OP_MATMUL_DQ;
  o.in = in;
  o.in2 = in2;
  o.out = out;
  o.M = tl.n / K;
  o.K = K;
  o.N = N;
  o.right_transpose = right_transpose != 0;
  o.q_group_size = q_group_size;
  o.dq_type = dq_type;
  o.dtype = tl.st == MI_ST_F16 ? MI_DT_F16 : MI_DT_BF16;
  // the launch checks type, group size and exactness limits: over no rows it does only that
  rc = matmul_dq_launch((const uint16_t *)tl.ptr(), (const uint16_t *)tr.ptr(), o.right_transpose, 0, K, N,
                        q_group_size, dq_type, o.dtype, (uint16_t *)to.ptr(), nullptr, m->stream);
  if (rc)
    return rc;
  m->ops.push_back(std::move(o));
  drop_graph(m);
  return MI_SUCCESS;
}

int mi_module_add_cast(mi_module *m, const char *input, const char *output, const mi_cast_attr *attr) {
  MI_REQUIRE(!m || !m->arena, MI_BAD_ARGUMENT, "mi_module: the memory plan is made; tensors and ops can no longer be added");
  int in, out, rc;
  if ((rc = find(m, input, &in)) || (rc = find(m, output, &out)))
    return rc;
  MI_REQUIRE(attr, MI_BAD_ARGUMENT, "mi_module_add_cast: null attribute");
  const Tensor &ti = m->tensors[in], &to = m->tensors[out];
  MI_REQUIRE(ti.st == attr->in_type && to.st == attr->out_type && ti.n == to.n, MI_BAD_ARGUMENT,
             "mi_module_add_cast: tensors do not match the cast's types or sizes");
  Op o;
  o.kind = OP_CAST;
  o.in = in;
  o.out = out;
  o.cast = *attr;
  o.cast.num_elem = ti.n;
  // validates the attribute and forms the per-call scalars exactly as mi_cast_launch does
  rc = cast_scalars(&o.cast, &o.inv_scale, &o.scale);
  if (rc)
    return rc;
  m->ops.push_back(std::move(o));
  drop_graph(m);
  return MI_SUCCESS;
}

int mi_module_set_tensor(mi_module *m, const char *name, const float *data, int64_t num_elem) {
  int idx, rc;
  if ((rc = find(m, name, &idx)))
    return rc;
  Tensor &t = m->tensors[idx];
  MI_REQUIRE(data && num_elem == t.n, MI_BAD_ARGUMENT, "mi_module_set_tensor: data size is not the tensor's");
  if (t.st == MI_ST_F32) {
    MI_HIP(hipMemcpyAsync(t.ptr(), data, (size_t)t.n * 4, hipMemcpyHostToDevice, m->stream));
    MI_HIP(hipStreamSynchronize(m->stream));
    return MI_SUCCESS;
  }
  if ((rc = need_staging(m, (size_t)t.n * 4)))
    return rc;
  MI_HIP(hipMemcpyAsync(m->staging.ptr, data, (size_t)t.n * 4, hipMemcpyHostToDevice, m->stream));
  mi_cast_attr c = plain_cast(MI_ST_F32, t.st, t.n);
  if ((rc = cast_launch(&c, m->staging.ptr, t.ptr(), t.n, 1.0f, 1.0f, false, m->stream)))
    return rc;
  MI_HIP(hipStreamSynchronize(m->stream));
  return MI_SUCCESS;
}

int mi_module_invoke(mi_module *m) {
  MI_REQUIRE(m, MI_BAD_ARGUMENT, "mi_module_invoke: null module");
  if (m->before || m->after) {  // hooks run on the host between launches: no graph replay
    const int rc = enqueue_range(m, 0, m->ops.size(), true);
    if (rc)
      return rc;
    MI_HIP(hipStreamSynchronize(m->stream));
    return MI_SUCCESS;
  }
  if (m->exec) {
    MI_HIP(hipGraphLaunch(m->exec, m->stream));
    MI_HIP(hipStreamSynchronize(m->stream));
    return MI_SUCCESS;
  }
  int rc = enqueue_all(m);
  if (rc)
    return rc;
  MI_HIP(hipStreamSynchronize(m->stream));
  // after the first (eager) pass: record the same launches into a graph when every op is a plain kernel launch
  if (!m->graph_tried) {
    m->graph_tried = true;
    bool ok = !m->ops.empty();
    for (const auto &o : m->ops)
      ok = ok && o.capturable;
    if (ok && hipStreamBeginCapture(m->stream, hipStreamCaptureModeThreadLocal) == hipSuccess) {
      rc = enqueue_all(m);
      hipGraph_t g = nullptr;
      hipError_t e = hipStreamEndCapture(m->stream, &g);
      if (rc == MI_SUCCESS && e == hipSuccess && g && hipGraphInstantiate(&m->exec, g, nullptr, nullptr, 0) == hipSuccess) {
        m->graph = g;
      } else {
        if (g)
          (void)hipGraphDestroy(g);
        m->exec = nullptr;
        (void)hipGetLastError();
      }
    }
  }
  return MI_SUCCESS;
}

static int get_tensor_impl(mi_module *m, const char *name, float *out, int64_t num_elem, bool scaled, const char *who) {
  int idx, rc;
  if ((rc = find(m, name, &idx)))
    return rc;
  Tensor &t = m->tensors[idx];
  MI_REQUIRE(out && num_elem == t.n, MI_BAD_ARGUMENT, std::string(who) + ": buffer size is not the tensor's");
  MI_REQUIRE(!t.shares_memory, MI_BAD_ARGUMENT,
             std::string(who) + ": '" + name + "' shares its memory with later tensors (mi_module_plan_memory); mark it "
             "as an output before planning to keep it");
  const void *src = t.ptr();
  if (t.st != MI_ST_F32) {
    if ((rc = need_staging(m, (size_t)t.n * 4)))
      return rc;
    mi_cast_attr c = plain_cast(t.st, MI_ST_F32, t.n);
    if ((rc = cast_launch(&c, t.ptr(), m->staging.ptr, t.n, 1.0f, 1.0f, false, m->stream)))
      return rc;
    src = m->staging.ptr;
  }
  MI_HIP(hipMemcpyAsync(out, src, (size_t)t.n * 4, hipMemcpyDeviceToHost, m->stream));
  MI_HIP(hipStreamSynchronize(m->stream));
  if (scaled && t.quant) {
    // py_cuda::cuda_to_host: 8-bit ((float)q - (float)zp) * (float)scale (pycuda.cpp:326-343); 16-bit q * scale with
    // the scale in double and no zero point (:370-379)
    if (t.st == MI_ST_I8 || t.st == MI_ST_U8) {
      const float zp = (float)t.q_zp, sc = (float)t.q_scale;
      for (int64_t i = 0; i < t.n; ++i)
        out[i] = (out[i] - zp) * sc;
    } else if (t.st == MI_ST_I16) {
      for (int64_t i = 0; i < t.n; ++i)
        out[i] = (float)((double)(int16_t)out[i] * t.q_scale);
    }
  }
  return MI_SUCCESS;
}

int mi_module_get_tensor(mi_module *m, const char *name, float *out, int64_t num_elem) {
  return get_tensor_impl(m, name, out, num_elem, true, "mi_module_get_tensor");
}

int mi_module_get_tensor_raw(mi_module *m, const char *name, float *out, int64_t num_elem) {
  return get_tensor_impl(m, name, out, num_elem, false, "mi_module_get_tensor_raw");
}

int mi_module_set_quant(mi_module *m, const char *name, double scale, int64_t zero_point) {
  int idx, rc;
  if ((rc = find(m, name, &idx)))
    return rc;
  Tensor &t = m->tensors[idx];
  MI_REQUIRE(t.st == MI_ST_I8 || t.st == MI_ST_U8 || t.st == MI_ST_I16, MI_BAD_ARGUMENT,
             "mi_module_set_quant: only 8-bit and int16 tensors carry a uniform quantization");
  t.quant = true;
  t.q_scale = scale;
  t.q_zp = zero_point;
  return MI_SUCCESS;
}

int mi_module_mark_output(mi_module *m, const char *name) {
  int idx, rc;
  if ((rc = find(m, name, &idx)))
    return rc;
  MI_REQUIRE(!m->arena, MI_BAD_ARGUMENT, "mi_module_mark_output: the memory plan is already made");
  m->tensors[idx].is_output = true;
  return MI_SUCCESS;
}

int mi_module_set_hooks(mi_module *m, mi_module_hook before, mi_module_hook after, void *user) {
  MI_REQUIRE(m, MI_BAD_ARGUMENT, "mi_module_set_hooks: null module");
  m->before = before;
  m->after = after;
  m->hook_user = user;
  return MI_SUCCESS;
}

int mi_module_invoke_at(mi_module *m, const char *name) {
  size_t op;
  int rc;
  MI_REQUIRE(m && name, MI_BAD_ARGUMENT, "mi_module_invoke_at: null argument");
  MI_REQUIRE(!m->arena, MI_BAD_ARGUMENT, "mi_module_invoke_at: not with a memory plan (the op's inputs may be gone)");
  if ((rc = find_op(m, name, &op)))
    return rc;
  if ((rc = enqueue_range(m, op, op + 1, true)))
    return rc;
  MI_HIP(hipStreamSynchronize(m->stream));
  return MI_SUCCESS;
}

int mi_module_invoke_from(mi_module *m, const char *name) {
  size_t op;
  int rc;
  MI_REQUIRE(m && name, MI_BAD_ARGUMENT, "mi_module_invoke_from: null argument");
  MI_REQUIRE(!m->arena, MI_BAD_ARGUMENT, "mi_module_invoke_from: not with a memory plan (earlier results may be gone)");
  if ((rc = find_op(m, name, &op)))
    return rc;
  if ((rc = enqueue_range(m, op, m->ops.size(), true)))
    return rc;
  MI_HIP(hipStreamSynchronize(m->stream));
  return MI_SUCCESS;
}

// Activation lifetimes.  The reference frees an activation on the GPU as soon as its last consumer has run
// (pycuda.cpp:633-660) and packs dead tensors' space on the host (host/ModuleInterpreter.cpp:86-232).  Freeing and
// allocating between launches is what a replayed graph cannot do, so the same saving is planned once: every
// intermediate (written by an op, not marked as an output) gets an offset in one arena, and two of them share bytes
// only when the launch that writes the later one comes after the last launch that reads the earlier one.
int mi_module_plan_memory(mi_module *m, int64_t *arena_bytes, int64_t *unplanned_bytes) {
  MI_REQUIRE(m, MI_BAD_ARGUMENT, "mi_module_plan_memory: null module");
  MI_REQUIRE(!m->arena, MI_BAD_ARGUMENT, "mi_module_plan_memory: already planned");
  const size_t n_t = m->tensors.size(), n_ops = m->ops.size();
  std::vector<int> launch_of(n_ops, 0);
  int n_launch = 0;
  for (size_t i = 0; i < n_ops;) {
    const size_t len = launch_len(m, i, n_ops);
    for (size_t k = 0; k < len; ++k)
      launch_of[i + k] = n_launch;
    ++n_launch;
    i += len;
  }
  std::vector<int> def(n_t, -1), last(n_t, -1);
  for (size_t i = 0; i < n_ops; ++i) {
    const Op &o = m->ops[i];
    if (def[o.out] < 0)
      def[o.out] = launch_of[i];
    last[o.out] = std::max(last[o.out], launch_of[i]);
    last[o.in] = std::max(last[o.in], launch_of[i]);
    if (o.in2 >= 0)
      last[o.in2] = std::max(last[o.in2], launch_of[i]);
  }
  struct Slot {
    int64_t off, bytes;
    int def, last;
  };
  std::vector<Slot> placed;
  std::vector<int64_t> offset(n_t, -1);
  int64_t extent = 0, separate = 0, summed = 0;
  // by definition order, first fit among the slots alive at the same time (256-byte granules keep every alignment)
  std::vector<int> order;
  for (size_t t = 0; t < n_t; ++t) {
    const Tensor &x = m->tensors[t];
    const int64_t bytes = ((x.n * st_bytes(x.st) + 255) / 256) * 256;
    if (def[t] < 0 || x.is_output) {  // inputs and outputs keep their own memory
      separate += bytes;
      continue;
    }
    order.push_back((int)t);
  }
  std::sort(order.begin(), order.end(), [&](int a, int b) { return def[a] < def[b] || (def[a] == def[b] && a < b); });
  for (int t : order) {
    const Tensor &x = m->tensors[t];
    const int64_t bytes = ((x.n * st_bytes(x.st) + 255) / 256) * 256;
    summed += bytes;
    std::vector<std::pair<int64_t, int64_t>> busy;
    for (const Slot &sl : placed)
      if (!(sl.last < def[t] || last[t] < sl.def))
        busy.push_back({sl.off, sl.off + sl.bytes});
    std::sort(busy.begin(), busy.end());
    int64_t off = 0;
    for (const auto &b : busy) {
      if (off + bytes <= b.first)
        break;
      off = std::max(off, b.second);
    }
    placed.push_back({off, bytes, def[t], last[t]});
    offset[t] = off;
    extent = std::max(extent, off + bytes);
  }
  if (extent > 0) {
    std::unique_ptr<DevMem> arena(new DevMem());
    int rc = arena->alloc((size_t)extent);
    if (rc)
      return rc;
    MI_HIP(hipStreamSynchronize(m->stream));
    drop_graph(m);  // a captured graph names the old addresses
    for (int t : order) {
      Tensor &x = m->tensors[t];
      x.planned = (char *)arena->ptr + offset[t];
      x.mem.reset();
      x.shares_memory = false;
    }
    for (size_t i = 0; i < placed.size(); ++i)
      for (size_t j = 0; j < placed.size(); ++j)
        if (i != j && placed[i].off < placed[j].off + placed[j].bytes && placed[j].off < placed[i].off + placed[i].bytes)
          m->tensors[order[i]].shares_memory = true;
    m->arena = std::move(arena);
  }
  if (arena_bytes)
    *arena_bytes = extent;
  if (unplanned_bytes)
    *unplanned_bytes = summed + separate;
  return MI_SUCCESS;
}

int mi_module_uses_graph(const mi_module *m) { return m && m->exec ? 1 : 0; }

}  // extern "C"
