// dvm::Kernel: graph building and the dtype lowering rules.
//
// The rules restate the reference's Kernel methods for a target without native
// bool / bf16 arithmetic (src/dvm.cc:1245-1447, GetBinaryS :586-676, PowS
// :255-279, NoLossCast :425-443, cast routing table :416-423): they fix the
// numerics of a graph (where values are rounded, which operations run in
// fp32), so they are kept operation for operation. int64 tensors, views,
// gathers and collectives are not implemented by this backend and raise.
#include <chrono>
#include <cmath>
#include <cstring>
#include <type_traits>

#include "ir.h"
#include "system.h"

namespace dvm {

// ---- fp16 / bf16 codecs -------------------------------------------------------

uint16_t F32ToF16Bits(float f) {
  uint32_t x;
  std::memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  x &= 0x7fffffffu;
  if (x >= 0x7f800000u) return static_cast<uint16_t>(sign | (x > 0x7f800000u ? 0x7e00u : 0x7c00u));
  if (x >= 0x477ff000u) return static_cast<uint16_t>(sign | 0x7c00u);  // rounds to infinity
  if (x < 0x38800000u) {
    // result is subnormal or zero: let an fp32 add do the round-to-nearest-even
    float v;
    std::memcpy(&v, &x, 4);
    float magic = 0.5f;  // 2^-1: adding it aligns the 10 result bits at the bottom of the mantissa
    v += magic;
    uint32_t r;
    std::memcpy(&r, &v, 4);
    return static_cast<uint16_t>(sign | (r - 0x3f000000u));
  }
  const uint32_t odd = (x >> 13) & 1u;
  x += 0xc8000fffu + odd;  // rebias the exponent (-112 << 23) and round to nearest even
  return static_cast<uint16_t>(sign | (x >> 13));
}

float F16BitsToF32(uint16_t h) {
  const uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16;
  uint32_t em = h & 0x7fffu;
  uint32_t out;
  if (em >= 0x7c00u) {
    out = sign | 0x7f800000u | ((em & 0x3ffu) << 13);
  } else if (em >= 0x0400u) {
    out = sign | ((em << 13) + 0x38000000u);
  } else if (em == 0) {
    out = sign;
  } else {
    // subnormal: value = em * 2^-24
    float v = static_cast<float>(em) * 5.9604644775390625e-08f;
    std::memcpy(&out, &v, 4);
    out |= sign;
  }
  float f;
  std::memcpy(&f, &out, 4);
  return f;
}

uint16_t F32ToBF16Bits(float f) {
  if (std::isnan(f)) return 0x7fc0u;
  uint32_t x;
  std::memcpy(&x, &f, 4);
  x += 0x7fffu + ((x >> 16) & 1u);
  return static_cast<uint16_t>(x >> 16);
}

float BF16BitsToF32(uint16_t h) {
  uint32_t x = static_cast<uint32_t>(h) << 16;
  float f;
  std::memcpy(&f, &x, 4);
  return f;
}

Float16::Float16(float v) : value_(F32ToF16Bits(v)) {}
Float16::Float16(int32_t v) : value_(F32ToF16Bits(static_cast<float>(v))) {}
Float16::operator float() const { return F16BitsToF32(value_); }
Float16::operator int32_t() const { return static_cast<int32_t>(F16BitsToF32(value_)); }
BFloat16::BFloat16(float v) : value_(F32ToBF16Bits(v)) {}
BFloat16::BFloat16(int32_t v) : value_(F32ToBF16Bits(static_cast<float>(v))) {}
BFloat16::operator float() const { return BF16BitsToF32(value_); }
BFloat16::operator int32_t() const { return static_cast<int32_t>(BF16BitsToF32(value_)); }

namespace {

float ScalarAsFloat(const ScalarRef &s) {
  switch (s.type) {
    case kFloat32: return s.f32;
    case kInt32: return static_cast<float>(s.i32);
    case kInt64: return static_cast<float>(s.i64);
    case kFloat16: return F16BitsToF32(s.f16);
    case kBFloat16: return BF16BitsToF32(s.f16);
    default: return 0.0f;
  }
}

uint32_t FloatBits(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  return u;
}

}  // namespace

uint32_t ScalarToContainer(const ScalarRef &s, DataType t, int half64) {
  if (half64 != 0) {  // one 32-bit word of an int64 scalar (whatever type it arrived as, converted like a C cast)
    int64_t v;
    switch (s.type) {
      case kInt64: v = s.i64; break;
      case kInt32: v = s.i32; break;
      default: v = static_cast<int64_t>(ScalarAsFloat(s)); break;
    }
    const uint64_t u = static_cast<uint64_t>(v);
    return static_cast<uint32_t>(half64 == 1 ? u : u >> 32);
  }
  switch (t) {
    case kFloat16: {
      if (s.type == kFloat16) return FloatBits(F16BitsToF32(s.f16));
      return FloatBits(F16BitsToF32(F32ToF16Bits(ScalarAsFloat(s))));
    }
    case kBFloat16: {
      if (s.type == kBFloat16) return FloatBits(BF16BitsToF32(s.f16));
      return FloatBits(BF16BitsToF32(F32ToBF16Bits(ScalarAsFloat(s))));
    }
    case kFloat32:
      return FloatBits(ScalarAsFloat(s));
    case kInt32: {
      int32_t v;
      if (s.type == kInt32) {
        v = s.i32;
      } else if (s.type == kInt64) {
        v = static_cast<int32_t>(s.i64);
      } else {
        v = static_cast<int32_t>(ScalarAsFloat(s));
      }
      return static_cast<uint32_t>(v);
    }
    case kBool:
      return FloatBits(ScalarAsFloat(s) != 0.0f ? 1.0f : 0.0f);
    default:
      Throw("scalar for an unsupported tensor type");
  }
}

// ---- Comm (single GPU: nothing to connect) ------------------------------------------

Comm::~Comm() {}
bool Comm::Init(int /*rank_id*/, int rank_size, int /*comm_type*/, const uint32_t * /*group_ranks*/) {
  return rank_size == 1;
}
void Comm::Init(void * /*hccl_comm*/) {}

// ---- Kernel ------------------------------------------------------------------------

namespace {

[[noreturn]] void Unsupported(const char *what) {
  Throw(std::string(what) + " is not supported by the gfx950 backend");
}

struct Operand {
  NDObject *obj = nullptr;
  ScalarOperand sc;
  bool IsObj() const { return obj != nullptr; }
};

template <typename T>
Operand MakeOperand(T v) {
  Operand o;
  if constexpr (std::is_same<T, NDObject *>::value) {
    o.obj = v;
  } else if constexpr (std::is_same<T, ScalarRef *>::value) {
    o.sc.ref = v;
  } else {
    o.sc.imm = v;
  }
  return o;
}

bool IsCompare(int op) { return op <= kLessEqual; }

// Intermediate type of one conversion step from `from` towards `to` (row = from, column = to).
const DataType kCastRoute[kDataTypeEnd][kDataTypeEnd] = {
    /* bool  */ {kBool, kFloat16, kFloat16, kFloat16, kFloat16, kFloat16},
    /* f16   */ {kBool, kFloat16, kFloat32, kFloat32, kInt32, kFloat32},
    /* bf16  */ {kFloat32, kFloat32, kBFloat16, kFloat32, kInt32, kFloat32},
    /* f32   */ {kFloat16, kFloat16, kBFloat16, kFloat32, kInt32, kInt64},
    /* i32   */ {kFloat16, kFloat16, kFloat32, kFloat32, kInt32, kInt64},
    /* i64   */ {kBool, kFloat32, kFloat32, kFloat32, kInt32, kInt64},
};

class Builder {
 public:
  explicit Builder(VKernel *k) : k_(k) {}

  NDObject *New(ObjKind kind, DataType t, NDObject *a = nullptr, NDObject *b = nullptr, NDObject *c = nullptr) {
    NDObject *o = new NDObject(kind, t);
    // A Store handed on as an operand (a later stage of a sequence kernel reading an earlier stage's
    // output, tests/ut/test_sequence_fusion.py:190-197) stands for the value it stores.
    // A Load bound to a Store by SetLoadBind reads what that Store writes: inside one kernel that is the value itself.
    auto value_of = [](NDObject *x) {
      if (x != nullptr && x->kind == kObjLoad && x->bound != nullptr) x = x->bound;
      return x != nullptr && x->kind == kObjStore ? x->in[0] : x;
    };
    o->in[0] = value_of(a);
    o->in[1] = value_of(b);
    o->in[2] = value_of(c);
    o->nin = c != nullptr ? 3 : (b != nullptr ? 2 : (a != nullptr ? 1 : 0));
    return k_->Append(o);
  }

  NDObject *CastStep(NDObject *x, DataType t, bool noloss) {
    NDObject *o = New(kObjCast, t, x);
    o->noloss_cast = noloss;
    return o;
  }

  // Conversion that cannot lose information on the values it is used for
  // (bool <-> arithmetic types); a cast back over such a cast is elided.
  NDObject *NoLossCast(NDObject *x, DataType t) {
    DataType cur = x->type_id_;
    while (cur != t) {
      const DataType step = kCastRoute[cur][t];
      if (x->kind == kObjCast && x->noloss_cast && x->in[0]->type_id_ == step) {
        x = x->in[0];
      } else {
        x = CastStep(x, step, true);
      }
      cur = step;
    }
    return x;
  }

  static bool IsBoolResult(const NDObject *x) {
    if (x->kind == kObjCompare || x->kind == kObjCompareS) return true;
    if (x->kind == kObjBinary) return x->op == kLogicalAnd || x->op == kLogicalOr;
    return false;
  }

  // ---- int64 tensors: pairs of int32 tensors (the reference's lowering, src/dvm.cc:478-760) ----
  // The 32-bit words of an int64 value: part 0 the low words, 1 the high words.
  NDObject *Half(NDObject *x, int part) {
    if (x->kind == kObjLoad && x->bound != nullptr) x = x->bound;
    if (x->kind == kObjStore) x = x->in[part];  // (a Store handed on as an operand stands for the value it stores)
    if (x->type_id_ == kInt32) return x;        // (the word itself: the store case above)
    if (x->kind == kObjPack64) return x->in[part];
    if (x->kind != kObjLoad) Throw("an int64 operand that is neither a Load nor the result of an int64 operator");
    for (auto it = k_->ops_.rbegin(); it != k_->ops_.rend(); ++it)  // one view per load and word, however often it is used
      if ((*it)->kind == kObjHalf64 && (*it)->in[0] == x && (*it)->op == part && (*it)->stage == k_->Stage()) return *it;
    NDObject *o = new NDObject(kObjHalf64, kInt32);
    o->in[0] = x;
    o->nin = 1;
    o->op = static_cast<uint8_t>(part);
    return k_->Append(o);
  }
  NDObject *Pack(NDObject *lo, NDObject *hi) { return New(kObjPack64, kInt64, lo, hi); }
  static ScalarOperand Imm32(int32_t v) {
    ScalarOperand s;
    s.imm = v;
    return s;
  }
  // (x <u y) on the bit patterns of two int32 tensors, as int32 0 / 1: both are moved by 2^31 first
  NDObject *UnsignedLess32(NDObject *x, NDObject *y) {
    NDObject *xb = NewBinaryS(kAdd, x, Imm32(INT32_MIN), false), *yb = NewBinaryS(kAdd, y, Imm32(INT32_MIN), false);
    return NoLossCast(TensorBinary(kLess, xb, yb), kInt32);
  }
  NDObject *Add64(NDObject *l, NDObject *r) {  // src/dvm.cc:678-689
    NDObject *llo = Half(l, 0), *rlo = Half(r, 0), *lhi = Half(l, 1), *rhi = Half(r, 1);
    NDObject *lo = TensorBinary(kAdd, llo, rlo);
    NDObject *carry = UnsignedLess32(lo, llo);
    return Pack(lo, TensorBinary(kAdd, TensorBinary(kAdd, lhi, rhi), carry));
  }
  NDObject *Sub64(NDObject *l, NDObject *r) {  // src/dvm.cc:691-702
    NDObject *llo = Half(l, 0), *rlo = Half(r, 0), *lhi = Half(l, 1), *rhi = Half(r, 1);
    NDObject *lo = TensorBinary(kSub, llo, rlo);
    NDObject *borrow = UnsignedLess32(llo, rlo);
    return Pack(lo, TensorBinary(kSub, TensorBinary(kSub, lhi, rhi), borrow));
  }
  NDObject *Compare64(int op, NDObject *l, NDObject *r) {  // src/dvm.cc:717-760
    NDObject *llo = Half(l, 0), *rlo = Half(r, 0), *lhi = Half(l, 1), *rhi = Half(r, 1);
    if (op == kEqual) return TensorBinary(kLogicalAnd, TensorBinary(kEqual, lhi, rhi), TensorBinary(kEqual, llo, rlo));
    if (op == kNotEqual) return TensorBinary(kLogicalOr, TensorBinary(kNotEqual, lhi, rhi), TensorBinary(kNotEqual, llo, rlo));
    // the high words decide, as signed numbers; where they are equal, the low words, as unsigned ones
    NDObject *lb = NewBinaryS(kAdd, llo, Imm32(INT32_MIN), false), *rb = NewBinaryS(kAdd, rlo, Imm32(INT32_MIN), false);
    NDObject *hi_cmp = NoLossCast(TensorBinary(op, lhi, rhi), kInt32);
    NDObject *hi_eq = NoLossCast(TensorBinary(kEqual, lhi, rhi), kInt32);
    NDObject *lo_cmp = NoLossCast(TensorBinary(op, lb, rb), kInt32);
    return NoLossCast(New(kObjSelect, kInt32, hi_eq, lo_cmp, hi_cmp), kBool);
  }
  // An int64 scalar as a tensor of the given shape (its two words as int32 fills; a ScalarRef is read again at
  // every code generation).
  NDObject *Fill64(const ScalarOperand &s, IntArrayRef *shape) {
    NDObject *w[2];
    for (int part = 0; part < 2; ++part) {
      w[part] = New(kObjBroadcastS, kInt32);
      w[part]->scalar = s;
      w[part]->aux_ref = shape;
      w[part]->half64 = static_cast<uint8_t>(part + 1);
    }
    return Pack(w[0], w[1]);
  }
  NDObject *ToInt64(NDObject *x) {
    if (x->type_id_ == kInt32) {  // sign extension: the high word is 0 - (x < 0)
      NDObject *neg = NoLossCast(ScalarBinary(kLess, Imm32(0), x, true), kInt32);
      return Pack(x, NewBinaryS(kAdd, NewBinaryS(kMul, neg, Imm32(-1), false), Imm32(0), false));
    }
    if (x->type_id_ != kFloat32) return ToInt64(Cast(x, x->type_id_ == kBool ? kInt32 : kFloat32));
    // fp32 -> int64 truncates toward zero (a C cast; magnitudes of 2^63 and above, infinities and NaN are undefined
    // there as well). |x| is split into its part above 2^32 and the rest, both exact in fp32; the low word goes
    // through the int32 conversion; a negative x negates the pair.
    ScalarOperand two32, inv32, two31, zero;
    two32.imm = 4294967296.0f;
    inv32.imm = 1.0f / 4294967296.0f;
    two31.imm = -2147483648.0f;
    zero.imm = 0.0f;
    NDObject *a = Unary(kAbs, Unary(kTrunc, x));
    NDObject *hi_f = Unary(kFloor, NewBinaryS(kMul, a, inv32, false));
    NDObject *lo_f = TensorBinary(kSub, a, NewBinaryS(kMul, hi_f, two32, false));
    // (the low part, in [0, 2^32), to its 32-bit pattern: below 2^31 the int32 conversion itself; from 2^31 on the
    // conversion of the value less 2^31, an exact subtraction there, moved back by an integer add)
    ScalarOperand pos31;
    pos31.imm = 2147483648.0f;
    NDObject *top = NoLossCast(ScalarBinary(kGreaterEqual, pos31, lo_f, true), kInt32);
    NDObject *lo_top = NewBinaryS(kAdd, Cast(NewBinaryS(kAdd, lo_f, two31, false), kInt32), Imm32(INT32_MIN), false);
    NDObject *lo = New(kObjSelect, kInt32, top, lo_top, Cast(lo_f, kInt32));
    NDObject *hi = Cast(hi_f, kInt32);
    // -(hi:lo) = (0 - lo) : (0 - hi - (lo != 0))
    NDObject *nlo = NewBinaryS(kAdd, NewBinaryS(kMul, lo, Imm32(-1), false), Imm32(0), false);
    NDObject *lo_nz = NoLossCast(ScalarBinary(kNotEqual, Imm32(0), lo, true), kInt32);
    NDObject *nhi = TensorBinary(kSub, NewBinaryS(kMul, hi, Imm32(-1), false), lo_nz);
    NDObject *is_neg = NoLossCast(ScalarBinary(kLess, zero, x, true), kInt32);
    return Pack(New(kObjSelect, kInt32, is_neg, nlo, lo), New(kObjSelect, kInt32, is_neg, nhi, hi));
  }
  NDObject *FromInt64(NDObject *x, DataType t) {
    NDObject *lo = Half(x, 0), *hi = Half(x, 1);
    if (t == kInt32) return lo;  // the low word: what a C cast keeps
    if (t == kBool) return TensorBinary(kLogicalOr, ScalarBinary(kNotEqual, Imm32(0), hi, true), ScalarBinary(kNotEqual, Imm32(0), lo, true));
    // to a float type, in fp32: the value is (high + [low < 0]) * 2^32 + low with the low word read as a signed
    // number, so that small magnitudes of either sign have a zero first term and come out exact; beyond 24
    // significant bits the two roundings of the sum can differ from one rounding of the value by a unit in the last
    // place.
    ScalarOperand two32;
    two32.imm = 4294967296.0f;
    NDObject *neg = Cast(NoLossCast(ScalarBinary(kLess, Imm32(0), lo, true), kInt32), kFloat32);
    NDObject *hi_f = TensorBinary(kAdd, Cast(hi, kFloat32), neg);
    NDObject *f = TensorBinary(kAdd, NewBinaryS(kMul, hi_f, two32, false), Cast(lo, kFloat32));
    return Cast(f, t);
  }

  NDObject *Cast(NDObject *x, DataType t) {
    if (x->type_id_ == t) return x;
    if (t == kInt64) return ToInt64(x);
    if (x->type_id_ == kInt64) return FromInt64(x, t);
    if (t == kBool && !IsBoolResult(x)) {
      ScalarOperand zero;
      zero.imm = 0;
      x = ScalarBinary(kNotEqual, zero, x, true);
    }
    DataType cur = x->type_id_;
    while (cur != t) {
      const DataType step = kCastRoute[cur][t];
      x = CastStep(x, step, false);
      cur = step;
    }
    return x;
  }

  NDObject *BroadcastScalar(const ScalarOperand &s, IntArrayRef *shape, DataType t) {
    if (t == kBool) return Cast(BroadcastScalar(s, shape, kFloat16), kBool);
    if (t == kInt64) return Fill64(s, shape);
    NDObject *o = New(kObjBroadcastS, t);
    o->scalar = s;
    o->aux_ref = shape;
    return o;
  }

  NDObject *Unary(int op, NDObject *x) {
    switch (x->type_id_) {
      case kBool: {
        NDObject *r = Unary(op, NoLossCast(x, kFloat16));
        return NoLossCast(r, kBool);
      }
      case kBFloat16:
        return Cast(Unary(op, Cast(x, kFloat32)), kBFloat16);
      case kFloat16:
        if (op >= kRound && op <= kTrunc) return Cast(Unary(op, Cast(x, kFloat32)), kFloat16);
        break;
      case kInt64:
        Unsupported("a unary operator on int64 tensors");
      default:
        break;
    }
    if (op == kLogicalNot) {
      ScalarOperand one;
      one.imm = 1;
      return ScalarBinaryOrFallback(kSub, one, x, false);
    }
    if (op == kReciprocal) {
      ScalarOperand one;
      one.imm = 1;
      return ScalarBinaryOrFallback(kDiv, one, x, false);
    }
    if (x->type_id_ == kInt32 && op != kAbs) Throw("unary operator without an int32 form");
    NDObject *o = New(kObjUnary, x->type_id_, x);
    o->op = static_cast<uint8_t>(op);
    return o;
  }

  NDObject *TensorBinary(int op, NDObject *l, NDObject *r) {
    switch (l->type_id_) {
      case kBool: {
        NDObject *res = TensorBinary(op, NoLossCast(l, kFloat16), NoLossCast(r, kFloat16));
        return NoLossCast(res, kBool);
      }
      case kBFloat16:
        if (op == kPow || op == kDiv) {
          return Cast(TensorBinary(op, Cast(l, kFloat32), Cast(r, kFloat32)), kBFloat16);
        }
        break;
      case kFloat16:
        if (op == kPow) return Cast(TensorBinary(op, Cast(l, kFloat32), Cast(r, kFloat32)), kFloat16);
        break;
      case kInt64:
        if (r->type_id_ != kInt64) Throw("int64 operator with an operand of another type");
        if (IsCompare(op)) return Compare64(op, l, r);
        if (op == kAdd) return Add64(l, r);
        if (op == kSub) return Sub64(l, r);
        Unsupported("this binary operator on int64 tensors");  // (the reference has add, sub and the compares: src/dvm.cc:1351-1364)
      default:
        break;
    }
    if (IsCompare(op)) {
      NDObject *o = New(kObjCompare, l->type_id_, l, r);
      o->op = static_cast<uint8_t>(op);
      return NoLossCast(o, kBool);
    }
    if (l->type_id_ == kInt32 && (op == kDiv || op == kPow)) Throw("binary operator without an int32 form");
    NDObject *o = New(kObjBinary, l->type_id_, l, r);
    o->op = static_cast<uint8_t>(op);
    return o;
  }

  NDObject *NewBinaryS(int op, NDObject *x, const ScalarOperand &s, bool scalar_left) {
    NDObject *o = New(kObjBinaryS, x->type_id_, x);
    o->op = static_cast<uint8_t>(op);
    o->scalar = s;
    o->scalar_left = scalar_left;
    return o;
  }

  // x ^ n for an integer n by repeated squaring.
  NDObject *PowInt(NDObject *x, const ScalarOperand &s, int32_t n) {
    uint32_t it = n < 0 ? 0u - static_cast<uint32_t>(n) : static_cast<uint32_t>(n);
    if (it == 0) {
      ScalarOperand one;
      one.imm = s.imm.type == kInt32 ? ScalarRef(1) : ScalarRef(1.0f);
      return BroadcastScalar(one, x->shape_ref_, x->type_id_);
    }
    NDObject *res = nullptr;
    if (it == 1) {
      res = New(kObjCopy, x->type_id_, x);
    } else {
      while (it != 0) {
        if (it & 1u) res = res == nullptr ? x : TensorBinary(kMul, res, x);
        if (it != 1) x = TensorBinary(kMul, x, x);
        it >>= 1;
      }
    }
    if (n < 0) res = Unary(kReciprocal, res);
    return res;
  }

  // Tensor (op) scalar when the operation has a scalar form; null otherwise.
  // rhs_val: the scalar is the right operand.
  NDObject *ScalarBinary(int op, const ScalarOperand &s, NDObject *x, bool rhs_val) {
    if (x->type_id_ == kInt64) {  // the scalar as a tensor of its two words, then the tensor form
      NDObject *b = Fill64(s, x->shape_ref_);
      return rhs_val ? TensorBinary(op, x, b) : TensorBinary(op, b, x);
    }
    const bool is_ref = s.ref != nullptr;
    switch (op) {
      case kAdd:
      case kMul:
      case kMinimum:
      case kMaximum:
        return NewBinaryS(op, x, s, false);
      case kDiv: {
        if (x->type_id_ == kBFloat16) return Cast(ScalarBinary(op, s, Cast(x, kFloat32), rhs_val), kBFloat16);
        if (x->type_id_ == kInt32) Throw("binary operator without an int32 form");
        return NewBinaryS(op, x, s, !rhs_val);
      }
      case kEqual:
      case kNotEqual:
      case kGreater:
      case kGreaterEqual:
      case kLess:
      case kLessEqual: {
        NDObject *o = New(kObjCompareS, x->type_id_, x);
        o->op = static_cast<uint8_t>(op);
        o->scalar = s;
        o->scalar_left = !rhs_val;
        return NoLossCast(o, kBool);
      }
      case kPow: {
        if (is_ref) return nullptr;
        const float v = ScalarAsFloat(s.imm);
        if (rhs_val) {
          const bool integral = s.imm.type == kInt32 || std::floor(v) == v;
          if (integral && std::fabs(v) < 2147483648.0f) return PowInt(x, s, static_cast<int32_t>(v));
          return nullptr;
        }
        if (v > 0.0f) {
          if (x->type_id_ != kFloat32) {
            ScalarOperand f;
            f.imm = v;
            const DataType orig = x->type_id_;
            return Cast(ScalarBinary(kPow, f, Cast(x, kFloat32), false), orig);
          }
          ScalarOperand lg;
          lg.imm = std::log(v);
          return Unary(kExp, NewBinaryS(kMul, x, lg, false));
        }
        return nullptr;
      }
      case kSub: {
        if (is_ref) return nullptr;
        ScalarOperand neg = s;
        if (rhs_val) {
          switch (neg.imm.type) {
            case kFloat32: neg.imm.f32 = -neg.imm.f32; break;
            case kInt32: neg.imm.i32 = static_cast<int32_t>(0u - static_cast<uint32_t>(neg.imm.i32)); break;
            case kInt64: neg.imm.i64 = -neg.imm.i64; break;
            default: neg.imm.f16 ^= 0x8000u; break;
          }
          return NewBinaryS(kAdd, x, neg, false);
        }
        ScalarOperand m1;
        switch (s.imm.type) {
          case kInt32: m1.imm = -1; break;
          case kInt64: m1.imm = static_cast<int64_t>(-1); break;
          case kFloat16: m1.imm = Float16(-1.0f); break;
          case kBFloat16: m1.imm = BFloat16(-1.0f); break;
          default: m1.imm = -1.0f; break;
        }
        return NewBinaryS(kAdd, NewBinaryS(kMul, x, m1, false), s, false);
      }
      default:
        return nullptr;
    }
  }

  NDObject *ScalarBinaryOrFallback(int op, const ScalarOperand &s, NDObject *x, bool rhs_val) {
    if (x->type_id_ == kBool) {
      NDObject *r = ScalarBinaryOrFallback(op, s, NoLossCast(x, kFloat16), rhs_val);
      return NoLossCast(r, kBool);
    }
    NDObject *o = ScalarBinary(op, s, x, rhs_val);
    if (o != nullptr) return o;
    NDObject *b = BroadcastScalar(s, x->shape_ref_, x->type_id_);
    return rhs_val ? TensorBinary(op, x, b) : TensorBinary(op, b, x);
  }

  NDObject *Binary(int op, const Operand &l, const Operand &r) {
    if (l.IsObj() && r.IsObj()) return TensorBinary(op, l.obj, r.obj);
    if (l.IsObj()) return ScalarBinaryOrFallback(op, r.sc, l.obj, true);
    if (r.IsObj()) return ScalarBinaryOrFallback(op, l.sc, r.obj, false);
    Throw("binary operator needs at least one tensor operand");
  }

 private:
  VKernel *k_;
};

}  // namespace

Kernel::Kernel() : kernel_(nullptr) {}
Kernel::~Kernel() { delete kernel_; }
Kernel &Kernel::operator=(Kernel &other) {
  if (this != &other) {
    delete kernel_;
    kernel_ = other.kernel_;
    other.kernel_ = nullptr;
  }
  return *this;
}
Kernel::Kernel(Kernel &other) : kernel_(other.kernel_) { other.kernel_ = nullptr; }

void Kernel::Reset(KernelType type, uint32_t flags) {
  g_system.Init();
  delete kernel_;
  switch (type) {
    case kVector:
    case kCube:
    case kMix:
    case kSplit:
    case kParallel:
    case kSequence:
    case kEager:  // operators are appended freely and cut into launches at code generation, exactly like kSplit:
                  // the reference's incremental cutting (src/xkernel.cc EagerKernel) and lazy code generation
                  // change when the work happens, not what is computed
      break;
    default:
      kernel_ = nullptr;
      Unsupported("this kernel type");
  }
  kernel_ = new VKernel(type, flags);
}

void Kernel::Clone(const Kernel &base, CloneHelper &helper) {
  VKernel *src = base.GetImpl();
  delete kernel_;
  kernel_ = new VKernel(src->KType(), src->Flags());
  for (NDObject *o : src->ops_) {
    NDObject *c = new NDObject(o->kind, o->type_id_);
    c->op = o->op;
    c->scalar_left = o->scalar_left;
    c->keepdims = o->keepdims;
    c->trans_a = o->trans_a;
    c->trans_b = o->trans_b;
    c->inplace = o->inplace;
    c->temp = o->temp;
    c->bound = o->bound != nullptr ? helper.GetClone(o->bound) : nullptr;
    c->noloss_cast = o->noloss_cast;
    c->half64 = o->half64;
    if (o->hi_view != nullptr) {
      c->hi_view = new NDObject(kObjStore, kInt32);
      c->hi_view->strided = true;
    }
    c->nin = o->nin;
    for (int i = 0; i < o->nin; ++i) c->in[i] = helper.GetClone(o->in[i]);
    c->scalar.imm = o->scalar.imm;
    c->scalar.ref = o->scalar.ref != nullptr ? helper.GetClone(o->scalar.ref) : nullptr;
    if (o->aux_ref == &o->own_axes_ref_) {  // a list the operator made for itself
      std::memcpy(c->own_axes_, o->own_axes_, sizeof(c->own_axes_));
      c->own_axes_ref_.data = c->own_axes_;
      c->own_axes_ref_.size = o->own_axes_ref_.size;
      c->aux_ref = &c->own_axes_ref_;
    } else {
      c->aux_ref = o->aux_ref != nullptr ? helper.GetClone(o->aux_ref) : nullptr;
    }
    c->elem_any = o->elem_any;
    c->gmm_type = o->gmm_type;
    c->gmm_sizes = o->gmm_sizes;
    c->group_list = o->group_list != nullptr ? helper.GetClone(o->group_list) : nullptr;
    c->pad_size = o->pad_size;
    c->scalar2.imm = o->scalar2.imm;
    c->scalar2.ref = o->scalar2.ref != nullptr ? helper.GetClone(o->scalar2.ref) : nullptr;
    c->addr = o->addr;
    c->strided = o->strided;
    c->view_offset = o->view_offset;
    c->stride_ref = o->stride_ref != nullptr ? helper.GetClone(o->stride_ref) : nullptr;
    c->full_shape_ref = o->full_shape_ref != nullptr ? helper.GetClone(o->full_shape_ref) : nullptr;
    c->slice_start = o->slice_start != nullptr ? helper.GetClone(o->slice_start) : nullptr;
    c->slice_end = o->slice_end != nullptr ? helper.GetClone(o->slice_end) : nullptr;
    c->slice_step = o->slice_step != nullptr ? helper.GetClone(o->slice_step) : nullptr;
    c->slice_dim = o->slice_dim;
    for (NDObject *p : o->parts) {  // parts precede their Concat, so their clones exist
      NDObject *pc = helper.GetClone(p);
      c->parts.push_back(pc);
      pc->cat = c;
    }
    c->dim_begin_ref = o->dim_begin_ref != nullptr ? helper.GetClone(o->dim_begin_ref) : nullptr;
    c->dim_end_ref = o->dim_end_ref != nullptr ? helper.GetClone(o->dim_end_ref) : nullptr;
    c->dim_begin = o->dim_begin;
    c->dim_end = o->dim_end;
    if (o->kind == kObjLoad && c->aux_ref != nullptr) c->shape_ref_ = c->aux_ref;
    kernel_->SetStage(o->stage);
    kernel_->Append(c);
    helper.SetClone(o, c);
  }
}

void Kernel::SetNameHint(const char *name, const char *fullname) {
  kernel_->name_ = name != nullptr ? name : "";
  kernel_->fullname_ = fullname != nullptr ? fullname : "";
}

NDObject *Kernel::Load(void *addr, IntArrayRef *shape, DataType type) {
  NDObject *o = new NDObject(kObjLoad, type);
  o->addr = addr;
  o->aux_ref = shape;
  o->shape_ref_ = shape;
  return kernel_->Append(o);
}

// Strided views (include/dvm.h:195-201 of the reference: Load with a stride list, SliceLoad, StridedSliceLoad,
// Store with a stride list). The innermost stride has to be 1: the VM reads and writes runs of consecutive
// elements; transposing views are rejected when the kernel is compiled.
NDObject *Kernel::Load(void *addr, IntArrayRef *shape, IntArrayRef *stride, DataType type) {
  NDObject *o = Load(addr, shape, type);
  if (stride != nullptr) {
    o->strided = true;
    o->stride_ref = stride;
  }
  return o;
}

// GlobalAccess names a tensor in memory for another operator to read (the index of a GatherLoad,
// include/dvm.h:284,297-307 of the reference). Here that is a Load: a load nothing reads costs nothing.
NDObject *Kernel::GlobalAccess(void *addr, IntArrayRef *shape, DataType type) { return Load(addr, shape, type); }

// GatherLoad (src/ops.h:632-657 of the reference; tests/ut/test_gather_load.py): the source tensor read at the
// positions an int32 index tensor names along one axis. Negative indices count from the end of the axis; indices past
// either end are clipped into it (the reference leaves them undefined).
NDObject *Kernel::GatherLoad(void *addr, IntArrayRef *shape, NDObject *index, int axis, DataType type, GatherMode gather_mode) {
  if (index == nullptr || index->type_id_ != kInt32) Throw("GatherLoad needs an int32 index tensor");
  if (type == kInt64) Throw("GatherLoad of int64 tensors is not supported by the gfx950 backend");
  NDObject *o = Builder(kernel_).New(kObjGather, type, index);
  o->addr = addr;
  o->full_shape_ref = shape;
  o->slice_dim = axis;
  o->op = gather_mode == kSliceGather ? 1 : 0;
  return o;
}
NDObject *Kernel::SliceLoad(void *addr, IntArrayRef *shape, IntArrayRef *start, IntArrayRef *size, DataType type) {
  NDObject *o = Load(addr, size, type);  // the value has the slice's shape
  o->strided = true;
  o->full_shape_ref = shape;
  o->slice_start = start;
  return o;
}
NDObject *Kernel::StridedSliceLoad(void *addr, IntArrayRef *shape, IntArrayRef *start, IntArrayRef *end, IntArrayRef *step,
                                   DataType type) {
  NDObject *o = Load(addr, shape, type);
  o->strided = true;
  o->full_shape_ref = shape;
  o->slice_start = start;
  o->slice_end = end;
  o->slice_step = step;
  o->aux_ref = nullptr;
  o->shape_ref_ = &o->own_ref_;  // the value's shape is computed from start / end / step
  return o;
}
NDObject *Kernel::MultiLoad(void *, IntArrayRef *, DataType, const Comm *) { Unsupported("MultiLoad"); }

NDObject *Kernel::Store(void *addr, NDObject *input) {
  Builder b(kernel_);
  if (input->type_id_ == kInt64) {
    // the two words of every element are stored through strides into one buffer (kObjStore with two inputs)
    NDObject *lo = b.Half(input, 0), *hi = b.Half(input, 1);
    if (lo->kind == kObjHalf64) lo = b.New(kObjCopy, kInt32, lo);
    if (hi->kind == kObjHalf64) hi = b.New(kObjCopy, kInt32, hi);
    NDObject *o = b.New(kObjStore, kInt64, lo, hi);
    o->addr = addr;
    o->strided = true;  // (nothing reads a value back from this buffer as if it were dense)
    o->hi_view = new NDObject(kObjStore, kInt32);
    o->hi_view->strided = true;
    return o;
  }
  if (input->IsLoad()) input = b.New(kObjCopy, input->type_id_, input);
  NDObject *o = b.New(kObjStore, input->type_id_, input);
  o->addr = addr;
  return o;
}

NDObject *Kernel::Store(void *addr, NDObject *input, IntArrayRef *stride) {
  NDObject *o = Store(addr, input);
  if (stride != nullptr && o->type_id_ == kInt64) {
    o->stride_ref = stride;  // (in int64 elements; Normalize doubles them)
  } else if (stride != nullptr) {
    o->strided = true;
    o->stride_ref = stride;
  }
  return o;
}

// PadStore (src/ops.h:713-731, src/ops.cc:1399-1412 of the reference): a store into a buffer whose innermost rows
// are pad_size elements longer than the value's; the padding is not written.
NDObject *Kernel::PadStore(void *addr, NDObject *input, int64_t pad_size) {
  if (pad_size < 0) Throw("PadStore needs a pad size of zero or more");
  if (input->type_id_ == kInt64) Throw("PadStore of int64 tensors is not supported by the gfx950 backend");
  NDObject *o = Store(addr, input);
  o->strided = true;
  o->pad_size = pad_size;
  return o;
}
void Kernel::SetStoreInplace(NDObject *store) { store->inplace = true; }
// A temporary Store and a Load bound to it hand a value from one part of a kernel to a later one through memory in
// the reference (src/dvm.cc:1583-1588). Here operators read the value directly (the launches are cut at code
// generation, and a value that crosses a cut gets its workspace there), so the bound Load stands for the stored value
// in every operator built after the binding, and a temporary Store that nothing else needs is dropped as dead code.
void Kernel::SetStoreTemp(NDObject *store) {
  if (store == nullptr || store->kind != kObjStore) Throw("SetStoreTemp needs a Store");
  store->temp = true;
}
void Kernel::SetLoadBind(NDObject *load, NDObject *access) {
  if (load == nullptr || load->kind != kObjLoad || load->strided) Throw("SetLoadBind needs a plain Load");
  if (access == nullptr || access->kind != kObjStore) Throw("SetLoadBind binds a Load to a Store of the same kernel");
  if (load->type_id_ != access->type_id_) Throw("SetLoadBind: the Load and the Store differ in type");
  for (NDObject *o : kernel_->ops_)
    for (int i = 0; i < o->nin; ++i)
      if (o->in[i] == load) Throw("SetLoadBind must come before the first use of the Load");
  load->bound = access;
}

NDObject *Kernel::_Unary(int op_type, NDObject *input) {
  if (op_type < 0 || op_type >= kUnaryTypeEnd) return nullptr;
  return Builder(kernel_).Unary(op_type, input);
}

template <UnaryType op_type>
NDObject *Kernel::Unary(NDObject *input) {
  return _Unary(op_type, input);
}

template <typename L, typename R>
NDObject *Kernel::_Binary(int op_type, L lhs, R rhs) {
  if (op_type < 0 || op_type >= kBinaryTypeEnd) return nullptr;
  return Builder(kernel_).Binary(op_type, MakeOperand(lhs), MakeOperand(rhs));
}

template <BinaryType op_type, typename L, typename R>
NDObject *Kernel::Binary(L lhs, R rhs) {
  return _Binary<L, R>(op_type, lhs, rhs);
}

#define DVM_INST_UNARY(op) template NDObject *Kernel::Unary<op>(NDObject *);
DVM_INST_UNARY(kSqrt) DVM_INST_UNARY(kAbs) DVM_INST_UNARY(kLog) DVM_INST_UNARY(kExp) DVM_INST_UNARY(kReciprocal)
DVM_INST_UNARY(kIsFinite) DVM_INST_UNARY(kLogicalNot) DVM_INST_UNARY(kRound) DVM_INST_UNARY(kFloor)
DVM_INST_UNARY(kCeil) DVM_INST_UNARY(kTrunc)
#undef DVM_INST_UNARY

#define DVM_INST_BINARY_T(L, R) template NDObject *Kernel::_Binary<L, R>(int, L, R);
DVM_INST_BINARY_T(NDObject *, NDObject *)
DVM_INST_BINARY_T(NDObject *, float) DVM_INST_BINARY_T(NDObject *, int32_t) DVM_INST_BINARY_T(NDObject *, int64_t)
DVM_INST_BINARY_T(NDObject *, Float16) DVM_INST_BINARY_T(NDObject *, BFloat16) DVM_INST_BINARY_T(NDObject *, ScalarRef *)
DVM_INST_BINARY_T(float, NDObject *) DVM_INST_BINARY_T(int32_t, NDObject *) DVM_INST_BINARY_T(int64_t, NDObject *)
DVM_INST_BINARY_T(Float16, NDObject *) DVM_INST_BINARY_T(BFloat16, NDObject *) DVM_INST_BINARY_T(ScalarRef *, NDObject *)
#undef DVM_INST_BINARY_T

#define DVM_INST_BINARY(op)                                              \
  template NDObject *Kernel::Binary<op>(NDObject *, NDObject *);         \
  template NDObject *Kernel::Binary<op>(NDObject *, float);              \
  template NDObject *Kernel::Binary<op>(NDObject *, int32_t);            \
  template NDObject *Kernel::Binary<op>(NDObject *, int64_t);            \
  template NDObject *Kernel::Binary<op>(NDObject *, Float16);            \
  template NDObject *Kernel::Binary<op>(NDObject *, BFloat16);           \
  template NDObject *Kernel::Binary<op>(NDObject *, ScalarRef *);        \
  template NDObject *Kernel::Binary<op>(float, NDObject *);              \
  template NDObject *Kernel::Binary<op>(int32_t, NDObject *);            \
  template NDObject *Kernel::Binary<op>(int64_t, NDObject *);            \
  template NDObject *Kernel::Binary<op>(Float16, NDObject *);            \
  template NDObject *Kernel::Binary<op>(BFloat16, NDObject *);           \
  template NDObject *Kernel::Binary<op>(ScalarRef *, NDObject *);
DVM_INST_BINARY(kEqual) DVM_INST_BINARY(kNotEqual) DVM_INST_BINARY(kGreater) DVM_INST_BINARY(kGreaterEqual)
DVM_INST_BINARY(kLess) DVM_INST_BINARY(kLessEqual) DVM_INST_BINARY(kAdd) DVM_INST_BINARY(kSub) DVM_INST_BINARY(kMul)
DVM_INST_BINARY(kDiv) DVM_INST_BINARY(kPow) DVM_INST_BINARY(kMaximum) DVM_INST_BINARY(kMinimum)
DVM_INST_BINARY(kLogicalAnd) DVM_INST_BINARY(kLogicalOr)
#undef DVM_INST_BINARY

NDObject *Kernel::_Reduce(int op_type, NDObject *input, IntArrayRef *dims, bool keepdims) {
  if (op_type == kSum && input->type_id_ != kFloat32) return nullptr;  // callers cast to fp32 first
  if (input->type_id_ == kInt64 || input->type_id_ == kBool) Throw("reduce over an unsupported tensor type");
  NDObject *o = Builder(kernel_).New(kObjReduce, input->type_id_, input);
  o->op = static_cast<uint8_t>(op_type);
  o->aux_ref = dims;
  o->keepdims = keepdims;
  return o;
}

NDObject *Kernel::Select(NDObject *cond, NDObject *lhs, NDObject *rhs) {
  Builder b(kernel_);
  if (lhs->type_id_ == kInt64) {  // word by word (src/dvm.cc:704-715)
    if (rhs->type_id_ != kInt64) Throw("select between an int64 tensor and one of another type");
    NDObject *c = b.NoLossCast(cond, kInt32);
    return b.Pack(b.New(kObjSelect, kInt32, c, b.Half(lhs, 0), b.Half(rhs, 0)), b.New(kObjSelect, kInt32, c, b.Half(lhs, 1), b.Half(rhs, 1)));
  }
  if (cond->type_id_ != lhs->type_id_) cond = b.NoLossCast(cond, lhs->type_id_);
  return b.New(kObjSelect, lhs->type_id_, cond, lhs, rhs);
}

NDObject *Kernel::Cast(NDObject *input, DataType type) { return Builder(kernel_).Cast(input, type); }

NDObject *Kernel::Broadcast(NDObject *input, IntArrayRef *shape) {
  Builder b(kernel_);
  if (input->type_id_ == kBool) {
    NDObject *r = Broadcast(b.NoLossCast(input, kFloat16), shape);
    return b.NoLossCast(r, kBool);
  }
  if (input->type_id_ == kInt64) return b.Pack(Broadcast(b.Half(input, 0), shape), Broadcast(b.Half(input, 1), shape));
  NDObject *o = b.New(kObjBroadcast, input->type_id_, input);
  o->aux_ref = shape;
  return o;
}

template <typename T>
NDObject *Kernel::Broadcast(T val, IntArrayRef *shape, DataType type) {
  return Builder(kernel_).BroadcastScalar(MakeOperand(val).sc, shape, type);
}
template NDObject *Kernel::Broadcast<float>(float, IntArrayRef *, DataType);
template NDObject *Kernel::Broadcast<int32_t>(int32_t, IntArrayRef *, DataType);
template NDObject *Kernel::Broadcast<int64_t>(int64_t, IntArrayRef *, DataType);
template NDObject *Kernel::Broadcast<Float16>(Float16, IntArrayRef *, DataType);
template NDObject *Kernel::Broadcast<BFloat16>(BFloat16, IntArrayRef *, DataType);
template NDObject *Kernel::Broadcast<ScalarRef *>(ScalarRef *, IntArrayRef *, DataType);

NDObject *Kernel::Reshape(NDObject *input, IntArrayRef *shape) {
  if (input->type_id_ == kInt64) {
    Builder b(kernel_);
    return b.Pack(Reshape(b.Half(input, 0), shape), Reshape(b.Half(input, 1), shape));
  }
  NDObject *o = Builder(kernel_).New(kObjReshape, input->type_id_, input);
  o->aux_ref = shape;
  return o;
}

NDObject *Kernel::Copy(NDObject *input) {
  Builder b(kernel_);
  if (input->type_id_ == kInt64) return b.Pack(Copy(b.Half(input, 0)), Copy(b.Half(input, 1)));
  return b.New(kObjCopy, input->type_id_, input);
}

NDObject *Kernel::MatMul(NDObject *lhs, NDObject *rhs, bool trans_a, bool trans_b, NDObject *bias) {
  if (lhs->type_id_ != rhs->type_id_ || (lhs->type_id_ != kFloat16 && lhs->type_id_ != kBFloat16)) {
    Throw("matmul needs two fp16 or two bf16 operands");
  }
  NDObject *o = Builder(kernel_).New(kObjMatMul, lhs->type_id_, lhs, rhs, bias);
  o->trans_a = trans_a;
  o->trans_b = trans_b;
  return o;
}

// Permute, Slice and Split are views: the input is kept (or written) in memory in its own layout and the
// consumers read it through the view's strides and offset; nothing is copied.
NDObject *Kernel::Permute(NDObject *input, IntArrayRef *dims) {
  if (input->type_id_ == kInt64) {
    Builder b(kernel_);
    return b.Pack(Permute(b.Half(input, 0), dims), Permute(b.Half(input, 1), dims));
  }
  NDObject *o = Builder(kernel_).New(kObjPermute, input->type_id_, input);
  o->aux_ref = dims;
  return o;
}
NDObject *Kernel::Slice(NDObject *input, IntArrayRef *start, IntArrayRef *size) {
  if (input->type_id_ == kInt64) {
    Builder b(kernel_);
    return b.Pack(Slice(b.Half(input, 0), start, size), Slice(b.Half(input, 1), start, size));
  }
  NDObject *o = Builder(kernel_).New(kObjSlice, input->type_id_, input);
  o->slice_start = start;
  o->aux_ref = size;
  return o;
}
NDObject *Kernel::Slice(NDObject *input, int dim, ScalarRef *begin, ScalarRef *end) {
  if (input->type_id_ == kInt64) {
    Builder b(kernel_);
    return b.Pack(Slice(b.Half(input, 0), dim, begin, end), Slice(b.Half(input, 1), dim, begin, end));
  }
  NDObject *o = Builder(kernel_).New(kObjSlice, input->type_id_, input);
  o->slice_dim = dim;
  o->dim_begin_ref = begin;
  o->dim_end_ref = end;
  return o;
}
// Concat: every input is written into its place in one buffer by the launch that computes it, the consumers read
// that buffer.
NDObject *Kernel::Concat(NDObject **inputs, size_t input_num, int dim) {
  if (input_num == 0) Throw("concat needs at least one input");
  Builder b(kernel_);
  if (inputs[0]->type_id_ == kInt64) {  // word by word
    std::vector<NDObject *> lo, hi;
    for (size_t i = 0; i < input_num; ++i) {
      if (inputs[i]->type_id_ != kInt64) Throw("concat inputs differ in type");
      lo.push_back(b.Half(inputs[i], 0));
      hi.push_back(b.Half(inputs[i], 1));
    }
    return b.Pack(Concat(lo.data(), input_num, dim), Concat(hi.data(), input_num, dim));
  }
  std::vector<NDObject *> parts;
  for (size_t i = 0; i < input_num; ++i) {
    if (inputs[i]->type_id_ != inputs[0]->type_id_) Throw("concat inputs differ in type");
    parts.push_back(b.New(kObjConcatPart, inputs[i]->type_id_, inputs[i]));
  }
  NDObject *o = b.New(kObjConcat, inputs[0]->type_id_);
  o->slice_dim = dim;
  o->parts = parts;
  for (NDObject *p : parts) p->cat = o;
  return o;
}
NDObject **Kernel::Split(NDObject *input, int dim, int64_t split_size, size_t split_num) {
  if (split_size <= 0 || split_num == 0) Throw("split needs a positive chunk size and count");
  NDObject **out = kernel_->NewObjectArray(split_num);
  for (size_t j = 0; j < split_num; ++j) {
    NDObject *o = Builder(kernel_).New(kObjSlice, input->type_id_, input);
    o->slice_dim = dim;
    o->dim_begin = static_cast<int64_t>(j) * split_size;
    o->dim_end = static_cast<int64_t>(j + 1) * split_size;  // clipped to the extent: the last chunk may be smaller
    out[j] = o;
  }
  return out;
}
// OneHot (include/dvm.h:482-491, src/ops.h:1333 of the reference; tests/ut/test_onehot.py): a dim of extent depth at
// position axis, on_value where the position equals the index, off_value elsewhere (also for indices outside [0, depth)).
template <typename T>
NDObject *Kernel::OneHot(NDObject *indices, IntArrayRef *depth, int axis, T on_value, T off_value) {
  if (indices == nullptr || indices->type_id_ != kInt32) Throw("OneHot needs int32 indices");
  DataType t = kFloat32;
  if constexpr (std::is_same<T, int32_t>::value) t = kInt32;
  if constexpr (std::is_same<T, Float16>::value) t = kFloat16;
  if constexpr (std::is_same<T, BFloat16>::value) t = kBFloat16;
  NDObject *o = Builder(kernel_).New(kObjOneHot, t, indices);
  o->aux_ref = depth;
  o->slice_dim = axis;
  o->scalar = MakeOperand(on_value).sc;
  o->scalar2 = MakeOperand(off_value).sc;
  return o;
}
template NDObject *Kernel::OneHot<float>(NDObject *, IntArrayRef *, int, float, float);
template NDObject *Kernel::OneHot<int32_t>(NDObject *, IntArrayRef *, int, int32_t, int32_t);
template NDObject *Kernel::OneHot<Float16>(NDObject *, IntArrayRef *, int, Float16, Float16);
template NDObject *Kernel::OneHot<BFloat16>(NDObject *, IntArrayRef *, int, BFloat16, BFloat16);
// ElemAny (src/ops.h:874-892, src/vm_aiv.cce:193-210 of the reference; tests/ut/test_element_any.py): one fp32 value,
// the maximum over every element of the input, so 1 when any element of a 0 / 1 mask is set. (The reference stores it
// only when it is not zero, into a buffer the caller has cleared; here it is always stored.)
NDObject *Kernel::ElemAny(NDObject *input) {
  if (input->type_id_ != kFloat32) Throw("ElemAny needs an fp32 input");
  kernel_->Normalize();  // (the input's rank)
  NDObject *o = Builder(kernel_).New(kObjReduce, kFloat32, input);
  o->op = static_cast<uint8_t>(kMax);
  const int r = o->in[0]->rank();
  for (int i = 0; i < r; ++i) o->own_axes_[i] = i;
  o->own_axes_ref_.data = o->own_axes_;
  o->own_axes_ref_.size = static_cast<size_t>(r);
  o->aux_ref = &o->own_axes_ref_;
  o->keepdims = false;
  o->elem_any = true;
  return o;
}
// GroupedMatMul (include/dvm.h:510-522, src/ops_m.cc:698-800 of the reference; tests/ut/test_gmm.py): the groups are
// ranges of the rows of lhs (kSplit_M: rhs is [groups, k, n], the result [m, n]) or of the k axis (kSplit_K: the result
// is [groups, m, n]); the list holds their upper bounds or their sizes and is read on the device at every launch.
NDObject *Kernel::GroupedMatMul(NDObject *lhs, NDObject *rhs, bool trans_a, bool trans_b, NDObject *bias, NDObject *group_list,
                                GmmSplitType group_type, GmmListType group_list_type) {
  if (group_type != kSplit_M && group_type != kSplit_K) Unsupported("GroupedMatMul over the n axis");
  if (group_list == nullptr || group_list->kind != kObjLoad || group_list->strided ||
      (group_list->type_id_ != kInt64 && group_list->type_id_ != kInt32)) {
    Throw("GroupedMatMul needs its group list as a plain Load of int64 or int32 values");
  }
  NDObject *o = MatMul(lhs, rhs, trans_a, trans_b, bias);
  o->gmm_type = group_type == kSplit_M ? 1 : 2;
  o->gmm_sizes = group_list_type == kListSize;
  o->group_list = group_list;
  return o;
}
NDObject *Kernel::_AllReduce(int, NDObject *, const Comm *) { Unsupported("AllReduce (single-GPU backend)"); }
NDObject *Kernel::AllGather(NDObject *, const Comm *) { Unsupported("AllGather (single-GPU backend)"); }
NDObject *Kernel::AllGatherV2(NDObject *, const Comm *) { Unsupported("AllGatherV2 (single-GPU backend)"); }
NDObject *Kernel::ReduceScatter(NDObject *, const Comm *) { Unsupported("ReduceScatter (single-GPU backend)"); }
NDObject *Kernel::ExtOut(NDObject *, int) { Unsupported("ExtOut"); }
// Stage boundary of a speculative vector kernel (kVector with kSpeculate). The reference tries to keep a reduce and its
// consumers in one kernel and falls back to a cut one when the reduced extent does not fit a tile
// (src/kernel.cc:2265-2578); the stage marker tells it where the cut would be. Here every vector kernel is compiled
// that way (a reduce and its consumers are consecutive sweeps of one launch whenever the schedule allows, separate
// launches otherwise), so the marker carries no information.
void Kernel::SpecNext() {
  if (!(kernel_->Flags() & kSpeculate)) Throw("SpecNext needs a kernel created with kSpeculate");
}

// Parallel and sequence kernels (src/xkernel.h, include/dvm.h:248-251 of the reference): the caller
// names the groups, every group becomes one or more launches of its own. The sub-kernel type and the
// core limit are advice for the reference's tile model; here the partitioner's own rules decide what
// a launch holds, and launches of one kernel run in stream order, which is a valid schedule for both.
void Kernel::ParallelAdd(KernelType type, uint32_t, size_t) {
  if (kernel_ == nullptr || kernel_->KType() != kParallel) Throw("ParallelAdd needs a kernel reset as kParallel");
  if (type != kVector && type != kCube && type != kMix) Unsupported("this sub-kernel type");
  kernel_->NextStage();
}
void Kernel::SequenceAdd(KernelType type, uint32_t) {
  if (kernel_ == nullptr || kernel_->KType() != kSequence) Throw("SequenceAdd needs a kernel reset as kSequence");
  if (type != kVector && type != kCube && type != kMix) Unsupported("this sub-kernel type");
  kernel_->NextStage();
}
void Kernel::Clear() {}

void Kernel::Normalize() { kernel_->Normalize(); }

size_t Kernel::PreCodeGen() {
  kernel_->Normalize();
  return kernel_->CodeGen(true);
}

void Kernel::CodeGen(const RelocEntry *relocs, size_t reloc_size, WsAllocator *ws_alloc) {
  const auto t0 = std::chrono::steady_clock::now();
  kernel_->CodeGen(false);
  kernel_->BindAddresses(relocs, reloc_size, ws_alloc, nullptr);
  kernel_->last_codegen_us_ =
      std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
}

int Kernel::Launch(void *stream) { return kernel_->Launch(stream); }

int Kernel::Launch(const RelocEntry *relocs, size_t reloc_size, void *workspace, void *stream) {
  kernel_->BindAddresses(relocs, reloc_size, nullptr, workspace);
  return kernel_->Launch(stream);
}

IntArrayRef *Kernel::GetShape(NDObject *op) { return op->shape_ref_; }
DataType Kernel::GetDType(NDObject *op) { return op->type_id_; }
const char *Kernel::Dump() const { return kernel_->DumpGraph(false).c_str(); }
const char *Kernel::DumpR() const { return kernel_->DumpGraph(true).c_str(); }
const char *Kernel::Das() const { return kernel_->DisAssemble().c_str(); }
const char *Kernel::Inspect() const { return kernel_->Inspect().c_str(); }

}  // namespace dvm
