// Flat C ABI + runner over dvm::Kernel (see include/dvm_c.h).
#include "../../../include/dvm_c.h"

#include <algorithm>
#include <chrono>
#include <cstring>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "ir.h"
#include "compiler.h"
#include "system.h"

using namespace dvm;

struct dvm_shape {
  std::vector<int64_t> dims;
  IntArrayRef ref;
  void Set(const int64_t *d, size_t n) {
    dims.assign(d, d + n);
    if (dims.capacity() < static_cast<size_t>(kMaxRank)) dims.reserve(kMaxRank);
    ref.data = dims.data();
    ref.size = dims.size();
  }
};

struct dvm_scalar {
  ScalarRef ref;
};

namespace {

thread_local std::string g_last_error;

struct Buffer {
  void *ptr = nullptr;
  size_t bytes = 0;
  bool owned = false;
};

struct WsAlloc : public WsAllocator {
  dvm_rt *rt;
  void *Alloc(size_t size) override;
};

}  // namespace

struct dvm_rt {
  Kernel kernel;
  KernelType ktype = kSplit;
  uint32_t flags = 0;
  bool das_mode = false;
  void *stream = nullptr;
  std::vector<std::unique_ptr<dvm_shape>> shapes;
  std::vector<std::unique_ptr<dvm_scalar>> scalars;
  std::vector<NDObject *> loads, stores;
  std::map<NDObject *, size_t> store_extent;  // strided stores: elements of the whole buffer they write into
  std::map<NDObject *, Buffer> buffers;
  Buffer workspace;
  dvm_ws_alloc_fn ws_fn = nullptr;  // the caller's workspace allocator (dvm_rt_set_workspace_allocator), or none
  void *ws_user = nullptr;
  std::map<NDObject *, std::unique_ptr<dvm_shape>> view_strides;  // loads bound through strides (dvm_rt_bind_device_view)
  uint64_t fake_addr = 0x1000;
  double jit_us = 0.0;
  WsAlloc ws_alloc;

  const DeviceApi &Api() const { return g_system.Api(); }

  void *AllocDevice(size_t bytes) {
    if (das_mode) {
      void *p = reinterpret_cast<void *>(fake_addr);
      fake_addr += (bytes + 0xfff) & ~static_cast<uint64_t>(0xfff);
      return p;
    }
    void *p = nullptr;
    int rc = Api().malloc(&p, bytes == 0 ? 16 : bytes);
    if (rc != 0) throw std::runtime_error(std::string("device allocation failed: ") + Api().error_string(rc));
    return p;
  }

  void Release(Buffer &b) {
    if (b.owned && b.ptr != nullptr && !das_mode) Api().free(b.ptr);
    b = Buffer();
  }

  void Ensure(NDObject *o, size_t bytes) {
    Buffer &b = buffers[o];
    if (b.ptr != nullptr && (!b.owned || b.bytes >= bytes)) return;
    Release(b);
    b.ptr = AllocDevice(bytes);
    b.bytes = bytes;
    b.owned = true;
  }

  void FreeAll() {
    for (auto &kv : buffers) Release(kv.second);
    buffers.clear();
    Release(workspace);
  }
};

namespace {

void *WsAlloc::Alloc(size_t size) {
  Buffer &w = rt->workspace;
  if (rt->ws_fn != nullptr && !rt->das_mode) {  // the caller's allocator: asked at every code generation, never freed here
    rt->Release(w);
    w.ptr = rt->ws_fn(size, rt->ws_user);
    if (w.ptr == nullptr) throw std::runtime_error("DVM EXCEPTION. reason: the workspace allocator returned no memory");
    w.bytes = size;
    w.owned = false;
    return w.ptr;
  }
  if (w.ptr == nullptr || w.bytes < size || !w.owned) {
    rt->Release(w);
    w.ptr = rt->AllocDevice(size);
    w.bytes = size;
    w.owned = true;
  }
  return w.ptr;
}

template <typename F>
auto Guard(F f, decltype(f()) on_error) -> decltype(f()) {
  try {
    return f();
  } catch (const std::exception &e) {
    g_last_error = e.what();
    return on_error;
  }
}

NDObject *Obj(dvm_obj *o) { return reinterpret_cast<NDObject *>(o); }
dvm_obj *Handle(NDObject *o) { return reinterpret_cast<dvm_obj *>(o); }

void ParseKernelType(const std::string &s, KernelType *type, uint32_t *flags) {
  std::string name = s, opts;
  auto pos = s.find(':');
  if (pos != std::string::npos) {
    name = s.substr(0, pos);
    opts = s.substr(pos + 1);
  }
  if (name.empty() || name == "vector") {
    *type = kVector;
  } else if (name == "split") {
    *type = kSplit;
  } else if (name == "mix") {
    *type = kMix;
  } else if (name == "cube") {
    *type = kCube;
  } else if (name == "parallel") {
    *type = kParallel;
  } else if (name == "seq") {
    *type = kSequence;
  } else if (name == "eager") {
    *type = kEager;
  } else {
    throw std::runtime_error("DVM EXCEPTION. reason: kernel type '" + name + "' is not supported by the gfx950 backend");
  }
  *flags = 0;
  size_t start = 0;
  while (start < opts.size()) {
    size_t end = opts.find(',', start);
    if (end == std::string::npos) end = opts.size();
    const std::string f = opts.substr(start, end - start);
    if (f == "dyn") {
      *flags |= kDynamic;
    } else if (f == "uws" || f == "unify_ws") {
      *flags |= kUnifyWS;
    } else if (f == "lazy") {
      *flags |= kLazyCodeGen;
    } else if (f == "spec" && *type == kVector) {
      *flags |= kSpeculate;
    } else if (f == "priv1" && *type == kVector) {  // with "spec": the stages are found automatically (no SpecNext calls)
      *flags |= kPrivate1;
    } else if (f == "priv1" || f == "priv2" || f == "opt_fractal") {
      // The reference picks between implementations of one kernel type with these (src/dvm.cc:1059-1106: the graph
      // kernel behind "split:priv1"; a fractal layout of its matrix unit), never between meanings: accepted, no effect.
    } else if (!f.empty()) {
      throw std::runtime_error("DVM EXCEPTION. reason: kernel flag '" + f + "' is not supported by the gfx950 backend");
    }
    start = end + 1;
  }
}

template <BinaryType kOp>
NDObject *BinaryDispatch(Kernel &k, const dvm_operand *l, const dvm_operand *r) {
  auto with_rhs = [&](auto lhs) -> NDObject * {
    switch (r->kind) {
      case 0: return k.Binary<kOp>(lhs, Obj(r->obj));
      default: throw std::runtime_error("DVM EXCEPTION. reason: binary operator needs a tensor operand");
    }
  };
  if (l->kind == 0) {
    NDObject *lhs = Obj(l->obj);
    switch (r->kind) {
      case 0: return k.Binary<kOp>(lhs, Obj(r->obj));
      case 1: return k.Binary<kOp>(lhs, static_cast<float>(r->f));
      case 2:  // (an integer that does not fit 32 bits travels as int64: it only means something to an int64 tensor)
        if (r->i != static_cast<int32_t>(r->i)) return k.Binary<kOp>(lhs, static_cast<int64_t>(r->i));
        return k.Binary<kOp>(lhs, static_cast<int32_t>(r->i));
      case 3: return k.Binary<kOp>(lhs, &r->ref->ref);
      default: break;
    }
  } else if (l->kind == 1) {
    return with_rhs(static_cast<float>(l->f));
  } else if (l->kind == 2) {
    if (l->i != static_cast<int32_t>(l->i)) return with_rhs(static_cast<int64_t>(l->i));
    return with_rhs(static_cast<int32_t>(l->i));
  } else if (l->kind == 3) {
    return with_rhs(&l->ref->ref);
  }
  throw std::runtime_error("DVM EXCEPTION. reason: bad operand kind");
}

}  // namespace

extern "C" {

const char *dvm_c_last_error(void) { return g_last_error.c_str(); }

dvm_rt *dvm_rt_new(const char *ker_type, const char *run_mode, int dev_id) {
  return Guard(
      [&]() -> dvm_rt * {
        std::unique_ptr<dvm_rt> rt(new dvm_rt());
        ParseKernelType(ker_type != nullptr ? ker_type : "", &rt->ktype, &rt->flags);
        const std::string mode = run_mode != nullptr ? run_mode : "dev";
        rt->das_mode = mode == "das";
        if (!rt->das_mode && mode != "dev") throw std::runtime_error("DVM EXCEPTION. reason: run mode '" + mode + "' is not supported");
        rt->ws_alloc.rt = rt.get();
        rt->kernel.Reset(rt->ktype, rt->flags);
        if (!rt->das_mode) {
          if (!g_system.HasDevice()) {
            throw std::runtime_error(std::string("DVM EXCEPTION. reason: no MI355X device layer: ") + g_system.LoadError());
          }
          // one device per process: the VM kernels and their limits were set up for it at the first use
          if (dev_id != g_system.device_id) {
            throw std::runtime_error("DVM EXCEPTION. reason: device " + std::to_string(dev_id) + " asked for, the backend runs on device " +
                                     std::to_string(g_system.device_id) + " (set DEVICE_ID before the first kernel)");
          }
          int rc = rt->Api().create_stream(&rt->stream);
          if (rc != 0) throw std::runtime_error(std::string("stream creation failed: ") + rt->Api().error_string(rc));
        }
        return rt.release();
      },
      nullptr);
}

void dvm_rt_delete(dvm_rt *rt) {
  if (rt == nullptr) return;
  rt->FreeAll();
  if (rt->stream != nullptr) rt->Api().destroy_stream(rt->stream);
  delete rt;
}

int dvm_rt_reset(dvm_rt *rt) {
  return Guard(
      [&]() {
        rt->FreeAll();
        rt->fake_addr = 0x1000;  // dry runs hand out the same placeholder addresses after every reset
        rt->store_extent.clear();
        rt->loads.clear();
        rt->stores.clear();
        rt->kernel.Reset(rt->ktype, rt->flags);
        return 0;
      },
      -1);
}

dvm_shape *dvm_rt_new_shape(dvm_rt *rt, const int64_t *dims, size_t n) {
  return Guard(
      [&]() {
        rt->shapes.emplace_back(new dvm_shape());
        rt->shapes.back()->dims.reserve(kMaxRank);
        rt->shapes.back()->Set(dims, n);
        return rt->shapes.back().get();
      },
      static_cast<dvm_shape *>(nullptr));
}

int dvm_shape_update(dvm_shape *s, const int64_t *dims, size_t n) {
  s->Set(dims, n);
  return 0;
}

dvm_scalar *dvm_rt_new_scalar(dvm_rt *rt, int dtype) {
  return Guard(
      [&]() {
        rt->scalars.emplace_back(new dvm_scalar());
        dvm_scalar *s = rt->scalars.back().get();
        if (dtype == kInt32) {
          s->ref = 0;
        } else if (dtype == kInt64) {
          s->ref = static_cast<int64_t>(0);
        } else {
          s->ref = 0.0f;
        }
        return s;
      },
      static_cast<dvm_scalar *>(nullptr));
}

int dvm_scalar_update_f(dvm_scalar *s, double v) {
  if (s->ref.type == kInt32) {
    s->ref = static_cast<int32_t>(v);
  } else if (s->ref.type == kInt64) {
    s->ref = static_cast<int64_t>(v);
  } else {
    s->ref = static_cast<float>(v);
  }
  return 0;
}

int dvm_scalar_update_i(dvm_scalar *s, int64_t v) {
  if (s->ref.type == kInt32) {
    s->ref = static_cast<int32_t>(v);
  } else if (s->ref.type == kInt64) {
    s->ref = v;
  } else {
    s->ref = static_cast<float>(v);
  }
  return 0;
}

dvm_obj *dvm_rt_load(dvm_rt *rt, dvm_shape *shape, int dtype) {
  return Guard(
      [&]() {
        NDObject *o = rt->kernel.Load(nullptr, &shape->ref, static_cast<DataType>(dtype));
        rt->loads.push_back(o);
        return Handle(o);
      },
      static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_store(dvm_rt *rt, dvm_obj *x) {
  return Guard(
      [&]() {
        NDObject *o = rt->kernel.Store(nullptr, Obj(x));
        rt->stores.push_back(o);
        return Handle(o);
      },
      static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_unary(dvm_rt *rt, int unary_type, dvm_obj *x) {
  return Guard(
      [&]() {
        NDObject *o = rt->kernel.Unary(unary_type, Obj(x));
        if (o == nullptr) throw std::runtime_error("DVM EXCEPTION. reason: bad unary operator");
        return Handle(o);
      },
      static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_binary(dvm_rt *rt, int binary_type, const dvm_operand *lhs, const dvm_operand *rhs) {
  return Guard(
      [&]() {
        Kernel &k = rt->kernel;
        NDObject *o = nullptr;
        switch (binary_type) {
          case kEqual: o = BinaryDispatch<kEqual>(k, lhs, rhs); break;
          case kNotEqual: o = BinaryDispatch<kNotEqual>(k, lhs, rhs); break;
          case kGreater: o = BinaryDispatch<kGreater>(k, lhs, rhs); break;
          case kGreaterEqual: o = BinaryDispatch<kGreaterEqual>(k, lhs, rhs); break;
          case kLess: o = BinaryDispatch<kLess>(k, lhs, rhs); break;
          case kLessEqual: o = BinaryDispatch<kLessEqual>(k, lhs, rhs); break;
          case kAdd: o = BinaryDispatch<kAdd>(k, lhs, rhs); break;
          case kSub: o = BinaryDispatch<kSub>(k, lhs, rhs); break;
          case kMul: o = BinaryDispatch<kMul>(k, lhs, rhs); break;
          case kDiv: o = BinaryDispatch<kDiv>(k, lhs, rhs); break;
          case kPow: o = BinaryDispatch<kPow>(k, lhs, rhs); break;
          case kMaximum: o = BinaryDispatch<kMaximum>(k, lhs, rhs); break;
          case kMinimum: o = BinaryDispatch<kMinimum>(k, lhs, rhs); break;
          case kLogicalAnd: o = BinaryDispatch<kLogicalAnd>(k, lhs, rhs); break;
          case kLogicalOr: o = BinaryDispatch<kLogicalOr>(k, lhs, rhs); break;
          default: throw std::runtime_error("DVM EXCEPTION. reason: bad binary operator");
        }
        return Handle(o);
      },
      static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_select(dvm_rt *rt, dvm_obj *cond, dvm_obj *lhs, dvm_obj *rhs) {
  return Guard([&]() { return Handle(rt->kernel.Select(Obj(cond), Obj(lhs), Obj(rhs))); }, static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_cast(dvm_rt *rt, dvm_obj *x, int dtype) {
  return Guard([&]() { return Handle(rt->kernel.Cast(Obj(x), static_cast<DataType>(dtype))); }, static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_broadcast(dvm_rt *rt, dvm_obj *x, dvm_shape *shape) {
  return Guard([&]() { return Handle(rt->kernel.Broadcast(Obj(x), &shape->ref)); }, static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_full(dvm_rt *rt, const dvm_operand *value, dvm_shape *shape, int dtype) {
  return Guard(
      [&]() {
        const DataType t = static_cast<DataType>(dtype);
        switch (value->kind) {
          case 1: return Handle(rt->kernel.Broadcast(static_cast<float>(value->f), &shape->ref, t));
          case 2:
            if (value->i != static_cast<int32_t>(value->i)) return Handle(rt->kernel.Broadcast(static_cast<int64_t>(value->i), &shape->ref, t));
            return Handle(rt->kernel.Broadcast(static_cast<int32_t>(value->i), &shape->ref, t));
          case 3: return Handle(rt->kernel.Broadcast(&value->ref->ref, &shape->ref, t));
          default: throw std::runtime_error("DVM EXCEPTION. reason: full needs a scalar value");
        }
      },
      static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_reshape(dvm_rt *rt, dvm_obj *x, dvm_shape *shape) {
  return Guard([&]() { return Handle(rt->kernel.Reshape(Obj(x), &shape->ref)); }, static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_reduce(dvm_rt *rt, int reduce_type, dvm_obj *x, dvm_shape *dims, int keepdims) {
  return Guard(
      [&]() {
        NDObject *o = rt->kernel.Reduce(reduce_type, Obj(x), &dims->ref, keepdims != 0);
        if (o == nullptr) throw std::runtime_error("DVM EXCEPTION. reason: sum needs an fp32 input (cast first)");
        return Handle(o);
      },
      static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_copy(dvm_rt *rt, dvm_obj *x) {
  return Guard([&]() { return Handle(rt->kernel.Copy(Obj(x))); }, static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_matmul(dvm_rt *rt, dvm_obj *lhs, dvm_obj *rhs, int trans_a, int trans_b, dvm_obj *bias) {
  return Guard(
      [&]() { return Handle(rt->kernel.MatMul(Obj(lhs), Obj(rhs), trans_a != 0, trans_b != 0, Obj(bias))); },
      static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_grouped_matmul(dvm_rt *rt, dvm_obj *lhs, dvm_obj *rhs, int trans_a, int trans_b, dvm_obj *bias, dvm_obj *group_list,
                               int group_type, int group_list_type) {
  return Guard(
      [&]() {
        if (group_type < 0 || group_type >= kGroupTypeEnd || group_list_type < 0 || group_list_type >= kEnd) {
          throw std::runtime_error("DVM EXCEPTION. reason: grouped_matmul: no such group type or list type");
        }
        return Handle(rt->kernel.GroupedMatMul(Obj(lhs), Obj(rhs), trans_a != 0, trans_b != 0, Obj(bias), Obj(group_list),
                                               static_cast<GmmSplitType>(group_type), static_cast<GmmListType>(group_list_type)));
      },
      static_cast<dvm_obj *>(nullptr));
}

// RtKernelPy::Clone (src/pybind_api.cc:923-993): rebuilds `base`'s graph in `rt`, with shapes, axis lists and
// scalars of its own, and translates the n handles in `items` (kinds: 0 operator, 1 shape, 2 scalar) to the
// clone's handles in `out`.
int dvm_rt_clone(dvm_rt *rt, dvm_rt *base, const int *kinds, void *const *items, size_t n, void **out) {
  return Guard(
      [&]() {
        struct Helper : public CloneHelper {
          IntArrayRef *GetClone(IntArrayRef *shape) override {
            auto it = shapes.find(shape);
            return it != shapes.end() ? it->second : shape;
          }
          ScalarRef *GetClone(ScalarRef *scalar) override {
            auto it = scalars.find(scalar);
            return it != scalars.end() ? it->second : scalar;
          }
          NDObject *GetClone(NDObject *op) override {
            auto it = ops.find(op);
            return it != ops.end() ? it->second : nullptr;
          }
          void SetClone(NDObject *op, NDObject *clone) override { ops[op] = clone; }
          std::map<IntArrayRef *, IntArrayRef *> shapes;
          std::map<ScalarRef *, ScalarRef *> scalars;
          std::map<NDObject *, NDObject *> ops;
        } helper;
        rt->FreeAll();
        rt->loads.clear();
        rt->stores.clear();
        std::map<const dvm_shape *, dvm_shape *> shape_of;
        std::map<const dvm_scalar *, dvm_scalar *> scalar_of;
        for (const auto &sh : base->shapes) {
          rt->shapes.emplace_back(new dvm_shape());
          rt->shapes.back()->dims.reserve(kMaxRank);
          rt->shapes.back()->Set(sh->dims.data(), sh->dims.size());
          helper.shapes[&sh->ref] = &rt->shapes.back()->ref;
          shape_of[sh.get()] = rt->shapes.back().get();
        }
        for (const auto &sc : base->scalars) {
          rt->scalars.emplace_back(new dvm_scalar());
          rt->scalars.back()->ref = sc->ref;
          helper.scalars[&sc->ref] = &rt->scalars.back()->ref;
          scalar_of[sc.get()] = rt->scalars.back().get();
        }
        rt->kernel.Clone(base->kernel, helper);
        for (NDObject *o : base->loads) rt->loads.push_back(helper.GetClone(o));
        for (NDObject *o : base->stores) rt->stores.push_back(helper.GetClone(o));
        for (size_t i = 0; i < n; ++i) {
          if (kinds[i] == 0) {
            out[i] = helper.GetClone(static_cast<NDObject *>(items[i]));
          } else if (kinds[i] == 1) {
            out[i] = shape_of[static_cast<const dvm_shape *>(items[i])];
          } else {
            out[i] = scalar_of[static_cast<const dvm_scalar *>(items[i])];
          }
          if (out[i] == nullptr) throw std::runtime_error("DVM EXCEPTION. reason: clone of a handle that does not belong to the base kernel");
        }
        return 0;
      },
      -1);
}

int dvm_rt_seq_add(dvm_rt *rt, int ktype, unsigned flags) {
  return Guard(
      [&]() {
        rt->kernel.SequenceAdd(static_cast<KernelType>(ktype), flags);
        return 0;
      },
      -1);
}

int dvm_rt_parallel_add(dvm_rt *rt, int ktype, unsigned flags, size_t core_limit) {
  return Guard(
      [&]() {
        rt->kernel.ParallelAdd(static_cast<KernelType>(ktype), flags, core_limit);
        return 0;
      },
      -1);
}

dvm_obj *dvm_rt_view_load(dvm_rt *rt, dvm_shape *shape, dvm_shape *stride, int dtype) {
  return Guard(
      [&]() {
        NDObject *o = rt->kernel.Load(nullptr, &shape->ref, &stride->ref, static_cast<DataType>(dtype));
        rt->loads.push_back(o);
        return Handle(o);
      },
      static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_slice_load(dvm_rt *rt, dvm_shape *shape, dvm_shape *start, dvm_shape *size, int dtype) {
  return Guard(
      [&]() {
        NDObject *o = rt->kernel.SliceLoad(nullptr, &shape->ref, &start->ref, &size->ref, static_cast<DataType>(dtype));
        rt->loads.push_back(o);
        return Handle(o);
      },
      static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_stridedslice_load(dvm_rt *rt, dvm_shape *shape, dvm_shape *start, dvm_shape *end, dvm_shape *step, int dtype) {
  return Guard(
      [&]() {
        NDObject *o = rt->kernel.StridedSliceLoad(nullptr, &shape->ref, &start->ref, &end->ref, &step->ref, static_cast<DataType>(dtype));
        rt->loads.push_back(o);
        return Handle(o);
      },
      static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_view_store(dvm_rt *rt, dvm_obj *x, dvm_shape *stride, size_t extent_elems) {
  return Guard(
      [&]() {
        NDObject *o = rt->kernel.Store(nullptr, Obj(x), &stride->ref);
        rt->stores.push_back(o);
        rt->store_extent[o] = extent_elems;
        return Handle(o);
      },
      static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_global_access(dvm_rt *rt, dvm_shape *shape, int dtype) { return dvm_rt_load(rt, shape, dtype); }

dvm_obj *dvm_rt_gather_load(dvm_rt *rt, dvm_shape *shape, dvm_obj *index, int dtype, int axis, int gather_mode) {
  return Guard(
      [&]() {
        NDObject *o = rt->kernel.GatherLoad(nullptr, &shape->ref, Obj(index), axis, static_cast<DataType>(dtype),
                                            gather_mode == 1 ? kSliceGather : kElementGather);
        rt->loads.push_back(o);  // the source tensor is bound to the operator like a load's
        return Handle(o);
      },
      static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_pad_store(dvm_rt *rt, dvm_obj *x, long long pad_size) {
  return Guard(
      [&]() {
        NDObject *o = rt->kernel.PadStore(nullptr, Obj(x), pad_size);
        rt->stores.push_back(o);
        return Handle(o);
      },
      static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_one_hot(dvm_rt *rt, dvm_obj *indices, dvm_shape *depth, int axis, double on_value, double off_value, int dtype) {
  return Guard(
      [&]() {
        switch (static_cast<DataType>(dtype)) {
          case kFloat32: return Handle(rt->kernel.OneHot(Obj(indices), &depth->ref, axis, static_cast<float>(on_value), static_cast<float>(off_value)));
          case kInt32: return Handle(rt->kernel.OneHot(Obj(indices), &depth->ref, axis, static_cast<int32_t>(on_value), static_cast<int32_t>(off_value)));
          case kFloat16: return Handle(rt->kernel.OneHot(Obj(indices), &depth->ref, axis, Float16(static_cast<float>(on_value)), Float16(static_cast<float>(off_value))));
          case kBFloat16: return Handle(rt->kernel.OneHot(Obj(indices), &depth->ref, axis, BFloat16(static_cast<float>(on_value)), BFloat16(static_cast<float>(off_value))));
          default: throw std::runtime_error("DVM EXCEPTION. reason: one_hot makes fp32, int32, fp16 or bf16 tensors");
        }
      },
      static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_element_any(dvm_rt *rt, dvm_obj *x) {
  return Guard([&]() { return Handle(rt->kernel.ElemAny(Obj(x))); }, static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_permute(dvm_rt *rt, dvm_obj *x, dvm_shape *dims) {
  return Guard([&]() { return Handle(rt->kernel.Permute(Obj(x), &dims->ref)); }, static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_slice(dvm_rt *rt, dvm_obj *x, dvm_shape *start, dvm_shape *size) {
  return Guard([&]() { return Handle(rt->kernel.Slice(Obj(x), &start->ref, &size->ref)); }, static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_slice_dim(dvm_rt *rt, dvm_obj *x, int dim, dvm_scalar *begin, dvm_scalar *end) {
  return Guard([&]() { return Handle(rt->kernel.Slice(Obj(x), dim, &begin->ref, &end->ref)); }, static_cast<dvm_obj *>(nullptr));
}

dvm_obj *dvm_rt_concat(dvm_rt *rt, dvm_obj **inputs, size_t n, int dim) {
  return Guard(
      [&]() {
        std::vector<NDObject *> objs;
        for (size_t i = 0; i < n; ++i) objs.push_back(Obj(inputs[i]));
        return Handle(rt->kernel.Concat(objs.data(), objs.size(), dim));
      },
      static_cast<dvm_obj *>(nullptr));
}

int dvm_rt_split(dvm_rt *rt, dvm_obj *x, int dim, long long chunk, size_t num, dvm_obj **out) {
  return Guard(
      [&]() {
        NDObject **parts = rt->kernel.Split(Obj(x), dim, chunk, num);
        for (size_t i = 0; i < num; ++i) out[i] = Handle(parts[i]);
        return 0;
      },
      -1);
}

int dvm_obj_set_view_offset(dvm_obj *io, long long elems) {
  Obj(io)->view_offset = elems;
  return 0;
}

int dvm_rt_set_store_inplace(dvm_rt *rt, dvm_obj *store) {
  return Guard(
      [&]() {
        rt->kernel.SetStoreInplace(Obj(store));
        return 0;
      },
      -1);
}

int dvm_rt_set_store_temp(dvm_rt *rt, dvm_obj *store) {
  return Guard(
      [&]() {
        rt->kernel.SetStoreTemp(Obj(store));
        return 0;
      },
      -1);
}

int dvm_rt_set_load_bind(dvm_rt *rt, dvm_obj *load, dvm_obj *store) {
  return Guard(
      [&]() {
        rt->kernel.SetLoadBind(Obj(load), Obj(store));
        return 0;
      },
      -1);
}

int dvm_rt_spec_next(dvm_rt *rt) {
  return Guard(
      [&]() {
        rt->kernel.SpecNext();
        return 0;
      },
      -1);
}

int dvm_obj_rank(const dvm_obj *o) { return reinterpret_cast<const NDObject *>(o)->rank(); }

int dvm_obj_shape(const dvm_obj *o, int64_t *dims, size_t cap) {
  const NDObject *n = reinterpret_cast<const NDObject *>(o);
  const size_t r = n->shape_ref_->size;
  for (size_t i = 0; i < r && i < cap; ++i) dims[i] = n->shape_ref_->data[i];
  return static_cast<int>(r);
}

int dvm_obj_dtype(const dvm_obj *o) { return reinterpret_cast<const NDObject *>(o)->type_id_; }

int dvm_rt_input(dvm_rt *rt, dvm_obj *load, const void *host, size_t bytes) {
  return Guard(
      [&]() {
        NDObject *o = Obj(load);
        // memory the caller bound earlier (dvm_rt_bind_device) is the caller's: host data never goes there
        auto bound = rt->buffers.find(o);
        if (bound != rt->buffers.end() && !bound->second.owned) bound->second = Buffer();
        rt->Ensure(o, bytes);
        if (!rt->das_mode && bytes > 0) {
          int rc = rt->Api().mem_to_dev(rt->buffers[o].ptr, host, bytes);
          if (rc != 0) throw std::runtime_error(std::string("host to device copy failed: ") + rt->Api().error_string(rc));
        }
        return 0;
      },
      -1);
}

int dvm_rt_bind_device(dvm_rt *rt, dvm_obj *io, void *device_ptr) {
  return Guard(
      [&]() {
        Buffer &b = rt->buffers[Obj(io)];
        rt->Release(b);
        b.ptr = device_ptr;
        b.owned = false;
        b.bytes = 0;
        return 0;
      },
      -1);
}

int dvm_rt_bind_device_view(dvm_rt *rt, dvm_obj *load, void *device_ptr, const int64_t *strides, size_t rank) {
  return Guard(
      [&]() {
        NDObject *o = Obj(load);
        if (o->kind != kObjLoad || o->full_shape_ref != nullptr) throw std::runtime_error("DVM EXCEPTION. reason: only a plain load takes a strided binding");
        if (strides == nullptr) {
          if (rt->view_strides.erase(o) != 0) {
            o->strided = false;
            o->stride_ref = nullptr;
          }
        } else {
          if (rank != static_cast<size_t>(o->shape_ref_->size)) throw std::runtime_error("DVM EXCEPTION. reason: one stride per dim of the load");
          std::unique_ptr<dvm_shape> &st = rt->view_strides[o];
          if (!st) st.reset(new dvm_shape());
          st->Set(strides, rank);
          o->strided = true;
          o->stride_ref = &st->ref;
          o->view_offset = 0;
        }
        Buffer &b = rt->buffers[o];
        rt->Release(b);
        b.ptr = device_ptr;
        b.owned = false;
        b.bytes = 0;
        return 0;
      },
      -1);
}

int dvm_rt_set_workspace_allocator(dvm_rt *rt, dvm_ws_alloc_fn alloc, void *user) {
  return Guard(
      [&]() {
        rt->ws_fn = alloc;
        rt->ws_user = user;
        if (!rt->workspace.owned) rt->workspace = Buffer();  // (memory of an earlier allocator is not ours to keep)
        return 0;
      },
      -1);
}

int dvm_rt_unbind_device(dvm_rt *rt) {
  return Guard(
      [&]() {
        for (auto &kv : rt->view_strides) {
          kv.first->strided = false;
          kv.first->stride_ref = nullptr;
        }
        rt->view_strides.clear();
        for (auto it = rt->buffers.begin(); it != rt->buffers.end();) {
          if (!it->second.owned) {
            it->first->addr = nullptr;
            it = rt->buffers.erase(it);
          } else {
            ++it;
          }
        }
        return 0;
      },
      -1);
}

int dvm_rt_normalize(dvm_rt *rt) {
  return Guard(
      [&]() {
        rt->kernel.Normalize();
        return 0;
      },
      -1);
}

int dvm_rt_codegen(dvm_rt *rt) {
  return Guard(
      [&]() {
        const auto t0 = std::chrono::steady_clock::now();
        rt->kernel.Normalize();
        const auto t1 = std::chrono::steady_clock::now();
        // outputs take their size from the inferred shapes
        for (NDObject *s : rt->stores) {
          if (s->temp) continue;  // SetStoreTemp: no output of the kernel
          auto ext = rt->store_extent.find(s);
          if (ext != rt->store_extent.end() || s->pad_size >= 0) {
            // a strided store writes part of a larger buffer, which starts out as zeros
            size_t elems = 0;
            if (s->pad_size >= 0) {  // PadStore: rows pad_size longer than the value's
              elems = s->rank() > 0 ? 1 : 0;
              for (int d = 0; d + 1 < s->rank(); ++d) elems *= static_cast<size_t>(s->dim(d));
              if (s->rank() > 0) elems *= static_cast<size_t>(s->dim(s->rank() - 1) + s->pad_size);
            } else {
              elems = ext->second;
            }
            const size_t bytes = elems * DTypeSize(s->type_id_);
            const bool fresh = rt->buffers.find(s) == rt->buffers.end() || rt->buffers[s].ptr == nullptr;
            rt->Ensure(s, bytes);
            if (fresh && !rt->das_mode && bytes > 0) {
              std::vector<char> zeros(bytes, 0);
              int rc = rt->Api().mem_to_dev(rt->buffers[s].ptr, zeros.data(), bytes);
              if (rc != 0) throw std::runtime_error(std::string("host to device copy failed: ") + rt->Api().error_string(rc));
            }
            continue;
          }
          const size_t bytes = static_cast<size_t>(s->numel()) * DTypeSize(s->type_id_);
          rt->Ensure(s, bytes);
        }
        std::vector<RelocEntry> relocs;
        relocs.reserve(rt->buffers.size());
        for (auto &kv : rt->buffers) relocs.emplace_back(kv.first, kv.second.ptr);
        for (NDObject *l : rt->loads) {
          if (l->bound != nullptr) continue;  // SetLoadBind: reads a value of the kernel, not memory of the caller
          if (rt->buffers.find(l) == rt->buffers.end()) throw std::runtime_error("DVM EXCEPTION. reason: a load has no input bound");
        }
        const auto t2 = std::chrono::steady_clock::now();
        rt->kernel.CodeGen(relocs.data(), relocs.size(), &rt->ws_alloc);
        const auto t3 = std::chrono::steady_clock::now();
        rt->jit_us = std::chrono::duration<double, std::micro>((t1 - t0) + (t3 - t2)).count();
        return 0;
      },
      -1);
}

double dvm_rt_jit_us(const dvm_rt *rt) { return rt->jit_us; }

int dvm_rt_run(dvm_rt *rt, void *stream, int flags) {
  return Guard(
      [&]() {
        if (rt->das_mode) return 0;
        void *s = (stream != nullptr || (flags & DVM_RUN_ON_GIVEN_STREAM) != 0) ? stream : rt->stream;
        int rc = rt->kernel.Launch(s);
        if (rc != 0) throw std::runtime_error(std::string("launch failed: ") + rt->Api().error_string(rc));
        if ((flags & DVM_RUN_WAIT) != 0) {
          rc = rt->Api().synchronize_stream(s);
          if (rc != 0) throw std::runtime_error(std::string("kernel execution failed: ") + rt->Api().error_string(rc));
        }
        return 0;
      },
      -1);
}

int dvm_rt_output(dvm_rt *rt, dvm_obj *store, void *host, size_t bytes) {
  return Guard(
      [&]() {
        if (rt->das_mode) {
          std::memset(host, 0, bytes);
          return 0;
        }
        auto it = rt->buffers.find(Obj(store));
        if (it == rt->buffers.end()) throw std::runtime_error("DVM EXCEPTION. reason: store has no buffer");
        if (bytes > 0) {
          int rc = rt->Api().mem_from_dev(host, it->second.ptr, bytes);
          if (rc != 0) throw std::runtime_error(std::string("device to host copy failed: ") + rt->Api().error_string(rc));
        }
        return 0;
      },
      -1);
}

void *dvm_rt_device_ptr(dvm_rt *rt, dvm_obj *io) {
  auto it = rt->buffers.find(Obj(io));
  return it == rt->buffers.end() ? nullptr : it->second.ptr;
}

namespace {
// warmup launches, then `iters` launches each bracketed by a pair of events on the runner's stream: microseconds per launch
std::vector<double> TimedLaunches(dvm_rt *rt, int warmup, int iters) {
  const DeviceApi &api = rt->Api();
  for (int i = 0; i < warmup; ++i) {
    int rc = rt->kernel.Launch(rt->stream);
    if (rc != 0) throw std::runtime_error(std::string("launch failed: ") + api.error_string(rc));
  }
  api.synchronize_stream(rt->stream);
  std::vector<void *> ev(2 * static_cast<size_t>(iters), nullptr);
  for (auto &e : ev) api.create_event(&e);
  int rc = 0;
  for (int i = 0; i < iters && rc == 0; ++i) {
    api.record_event(ev[2 * i], rt->stream);
    rc = rt->kernel.Launch(rt->stream);
    api.record_event(ev[2 * i + 1], rt->stream);
  }
  const int rs = api.synchronize_stream(rt->stream);
  std::vector<double> us(static_cast<size_t>(iters), 0.0);
  for (int i = 0; i < iters && rc == 0 && rs == 0; ++i) {
    float ms = 0.0f;
    api.event_elapsed_time(&ms, ev[2 * i], ev[2 * i + 1]);
    us[i] = ms * 1000.0;
  }
  for (auto &e : ev) api.destroy_event(e);
  if (rc != 0) throw std::runtime_error(std::string("launch failed: ") + api.error_string(rc));
  if (rs != 0) throw std::runtime_error(std::string("kernel execution failed: ") + api.error_string(rs));
  return us;
}
}  // namespace

int dvm_rt_perf(dvm_rt *rt, int warmup, int iters, double out[3]) {
  return Guard(
      [&]() {
        out[0] = out[1] = out[2] = 0.0;
        if (rt->das_mode || iters <= 0) return 0;
        const std::vector<double> us = TimedLaunches(rt, warmup, iters);
        double mn = 1e30, mx = 0.0, sum = 0.0;
        for (double v : us) {
          mn = std::min(mn, v);
          mx = std::max(mx, v);
          sum += v;
        }
        out[0] = mn;
        out[1] = mx;
        out[2] = sum / iters;
        return 0;
      },
      -1);
}

void dvm_set_online_tuner(int enable) {
  g_system.Init();
  if (enable) g_system.SetOnlineTuner();
  else g_system.UnsetOnlineTuner();
}
void dvm_set_lazy_tuner(int enable) {
  g_system.Init();
  if (enable) g_system.SetLazyTuner();
  else g_system.UnsetLazyTuner();
}
void dvm_tuner_stats(uint64_t *shapes_measured, uint64_t *table_size) { CubeTunerStats(shapes_measured, table_size); }
void dvm_tuner_clear(void) { CubeTunerClear(); }

int dvm_rt_perf_samples(dvm_rt *rt, int warmup, int iters, double *samples) {
  return Guard(
      [&]() {
        for (int i = 0; i < iters; ++i) samples[i] = 0.0;
        if (rt->das_mode || iters <= 0) return 0;
        const std::vector<double> us = TimedLaunches(rt, warmup, iters);
        for (int i = 0; i < iters; ++i) samples[i] = us[i];
        return 0;
      },
      -1);
}

int dvm_rt_num_launches(const dvm_rt *rt) {
  int n = 0;
  for (const Program &p : rt->kernel.GetImpl()->programs_) n += (p.skip ? 0 : 1) + static_cast<int>(p.fills.size());
  return n;
}

size_t dvm_rt_workspace_bytes(const dvm_rt *rt) { return rt->kernel.GetImpl()->ws_bytes_; }

int dvm_rt_program_count(const dvm_rt *rt) { return static_cast<int>(rt->kernel.GetImpl()->programs_.size()); }

int dvm_rt_program(dvm_rt *rt, int i, void *blob, uint32_t geometry[3], uint32_t *ws_words, size_t cap) {
  return Guard(
      [&]() {
        VKernel *k = rt->kernel.GetImpl();
        if (i < 0 || i >= static_cast<int>(k->programs_.size())) throw std::runtime_error("DVM EXCEPTION. reason: no such launch");
        const Program &p = k->programs_[i];
        if (!p.fills.empty()) throw std::runtime_error("DVM EXCEPTION. reason: this launch needs a buffer cleared first and cannot be exported");
        VmParam copy = p.blob;
        int n = 0;
        geometry[0] = geometry[1] = geometry[2] = 0;
        if (!p.skip) {
          geometry[0] = p.grid;
          geometry[1] = p.threads;
          geometry[2] = p.lds_bytes;
          for (const Program::Patch &pt : p.patches) {
            if (pt.op_id >= 0 || pt.ws_slot < 0) continue;
            copy.w[pt.word] = k->ws_offsets_[pt.ws_slot] + static_cast<uint64_t>(pt.byte_offset);
            if (static_cast<size_t>(n) < cap) ws_words[n] = pt.word;
            ++n;
          }
        }
        std::memcpy(blob, &copy, sizeof(copy));
        return n;
      },
      -1);
}

const char *dvm_rt_das(dvm_rt *rt) {
  return Guard([&]() { return rt->kernel.Das(); }, static_cast<const char *>(nullptr));
}
const char *dvm_rt_dump(dvm_rt *rt) {
  return Guard([&]() { return rt->kernel.Dump(); }, static_cast<const char *>(nullptr));
}
const char *dvm_rt_dump_r(dvm_rt *rt) {
  return Guard([&]() { return rt->kernel.DumpR(); }, static_cast<const char *>(nullptr));
}
const char *dvm_rt_inspect(dvm_rt *rt) {
  return Guard([&]() { return rt->kernel.Inspect(); }, static_cast<const char *>(nullptr));
}

void dvm_c_f32_to_bf16(const float *src, uint16_t *dst, size_t n) {
  for (size_t i = 0; i < n; ++i) dst[i] = F32ToBF16Bits(src[i]);
}
void dvm_c_bf16_to_f32(const uint16_t *src, float *dst, size_t n) {
  for (size_t i = 0; i < n; ++i) dst[i] = BF16BitsToF32(src[i]);
}

int dvm_c_has_device(void) {
  g_system.Init();
  return g_system.HasDevice() ? 1 : 0;
}
int dvm_c_core_num(void) {
  g_system.Init();
  return static_cast<int>(g_system.core_num);
}

}  // extern "C"
