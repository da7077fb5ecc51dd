// Operator layer of the spatial path: the graph core the ops plug into, and the eight ops of
// the path with the reference's names, factories and _forward/_backward entry points.
//
// Mirrors include/arraydiff/op.hh + src/op.cc of the reference for this path only:
//   ids and traversal        op.hh:40-169, 593-683   (NodeId/TxnId/EpochId, OperatorStack, Op)
//   TxnVar / VarData / Var   op.hh:171-591, 685-697  (first-touch-per-transaction buffers)
//   SpatialScatter2DOp       op.hh:2175-2263, op.cc:2383-2468
//   SpatialGather2DOp        op.hh:2265-2353, op.cc:2470-2553
//   HaloPad2DOp              op.hh:2355-2453, op.cc:2555-2712
//   HaloUnpad2DOp            op.hh:2455-2545, op.cc:2714-2870
//   HaloRepad2DOp            op.hh:2547-2643, op.cc:2872-2960  (forward only, as in the reference)
//   HaloExch2DOp             op.hh:2645-2709, op.cc:2962-3052
//   CudnnConv2DOp            op.hh:1799-1940, op.cc:1343-1727  (here SlabConv2DOp; the old name is an alias)
//   CudnnSoftmaxNLLLossOp    op.hh:3380-3459, op.cc:4112-4188  (here SoftmaxNLLLossOp; alias kept)
// The write protocol is the reference's: overwrite() = one exclusive writer per transaction;
// accumulate(init_fn) = the first toucher in a transaction runs init_fn (zeroing), every node
// adds once.  Buffers are allocated on first write and shared by clones of a VarData.
// All arithmetic is behind the C ABI (adh_capi.h); nothing here launches a kernel itself.
#ifndef ARRAYDIFF_OP_HH
#define ARRAYDIFF_OP_HH

#include "arraydiff/array_gpu.hh"
#include "arraydiff/context.hh"
#include "arraydiff/spatial.hh"

#include <array>
#include <cassert>
#include <cmath>
#include <functional>
#include <map>
#include <memory>
#include <random>
#include <set>
#include <type_traits>
#include <vector>

namespace arraydiff {

using std::array;
using std::function;
using std::make_shared;
using std::shared_ptr;
using std::vector;

// ---------------------------------------------------------------------------
// ids (thread-local counters, op.cc:77-110)
// ---------------------------------------------------------------------------
uint64_t next_raw_id(int kind);

template <int Kind>
class RawId {
public:
  RawId() : id_(next_raw_id(Kind)) {}
  uint64_t raw_id() const { return id_; }
  bool operator==(const RawId &o) const { return id_ == o.id_; }

private:
  uint64_t id_;
};
typedef RawId<0> NodeId;
typedef RawId<1> EpochId;
typedef RawId<2> TxnId;
typedef RawId<3> VarId;

// A read/write hazard the reference would assert on (op.hh:249-478).
class HazardError : public std::logic_error {
public:
  explicit HazardError(const std::string &w) : std::logic_error(w) {}
};

// A set of variables to persist, load or store as one flat vector (op.hh:110-171).  While a walk
// over the graph holds the lock, mask() lets every member through exactly once, so a variable
// that several nodes share lands in the flat vector one time.
class VarIdSet {
public:
  static VarIdSet Singleton(VarId v) {
    VarIdSet s;
    s.insert(v);
    return s;
  }
  void insert(VarId v) {
    if (locked_) throw HazardError("VarIdSet: insert while a walk holds the set");
    ids_.insert(v.raw_id());
  }
  void insert_all(const VarIdSet &o) {
    if (locked_) throw HazardError("VarIdSet: insert while a walk holds the set");
    ids_.insert(o.ids_.begin(), o.ids_.end());
  }
  bool contains(VarId v) const { return ids_.count(v.raw_id()) != 0; }
  size_t size() const { return ids_.size(); }
  void lock() {
    if (locked_) throw HazardError("VarIdSet: already locked");
    seen_.clear();
    locked_ = true;
  }
  void unlock() {
    locked_ = false;
    seen_.clear();
  }
  bool mask(VarId v) {
    if (!locked_) throw HazardError("VarIdSet: mask outside a walk");
    if (!ids_.count(v.raw_id())) return false;
    return seen_.insert(v.raw_id()).second;
  }

private:
  bool locked_ = false;
  std::set<uint64_t> ids_, seen_;
};

// ---------------------------------------------------------------------------
// TxnVar: one buffer, (re)initialised per transaction
// ---------------------------------------------------------------------------
template <typename V>
struct IsBatchArray : std::false_type {};
template <typename Dim, typename T>
struct IsBatchArray<GPUBatchArray<Dim, T>> : std::true_type {};

template <typename V>
class TxnVar {
public:
  typedef typename V::Shape VShape;
  typedef typename V::Ctx Ctx;

  TxnVar() {}
  explicit TxnVar(VShape shape, size_t batch_shape = 0)
      : shape_(shape), offset_(VShape::Zero()), stride_(shape.packed_stride()), batch_shape_(batch_shape),
        buf_(make_shared<Buf>()) {}
  TxnVar(VShape shape, VShape offset, VShape stride, size_t batch_shape)
      : shape_(shape), offset_(offset), stride_(stride), batch_shape_(batch_shape), buf_(make_shared<Buf>()) {}

  TxnVar clone() const { return *this; }  // shares the buffer
  VarId var() const { return buf().var; }
  // Not in the reference.  From now on this variable (and every copy of it that a node already holds) IS `target`:
  // one buffer, one transaction state.  Both must have one layout.
  void forward_to(TxnVar &target) {
    if (target.shape_ != shape_ || target.offset_ != offset_ || target.stride_ != stride_ || target.batch_shape_ != batch_shape_)
      throw std::invalid_argument("TxnVar::forward_to: the two variables must have one layout");
    shared_ptr<Buf> mine = root(), theirs = target.root();
    if (mine == theirs) return;
    if (mine->buffer) throw HazardError("TxnVar::forward_to after the buffer was allocated");
    mine->forward = theirs;
  }
  VShape shape() const { return shape_; }
  VShape offset() const { return offset_; }
  VShape stride() const { return stride_; }
  size_t batch_shape() const { return batch_shape_; }

  // Exclusive write.  true: the caller is (or becomes) the only writer of this transaction
  // and must produce the value; false: another node already produced it.
  bool overwrite(TxnId txn, NodeId node, Ctx *ctx) {
    begin(txn, ctx);
    Buf &b = buf();
    if (b.readers.count(node.raw_id())) throw HazardError("overwrite after read by the same node");
    if (!b.writers.empty() && !b.writers.count(node.raw_id())) return false;
    b.writers.insert(node.raw_id());
    b.all_zero = false;
    return true;
  }
  // Accumulating write.  The first toucher of a transaction runs init_fn on the buffer; the
  // return value says whether THIS node still has to add its contribution.
  bool accumulate(TxnId txn, NodeId node, Ctx *ctx, function<void(V *)> init_fn) {
    const bool fresh = begin(txn, ctx);
    Buf &b = buf();
    if (fresh) init_fn(b.buffer.get());
    if (b.writers.count(node.raw_id())) return false;
    b.writers.insert(node.raw_id());
    b.all_zero = false;
    return true;
  }
  // Not in the reference.  True while the buffer is known to hold nothing but zeros: it was allocated (cleared) or
  // a writer declared it so, and no write access has been handed out since.  A node that would clear the buffer
  // again can skip the fill.
  bool known_zero() const { return buf().buffer && buf().all_zero; }
  // a writer of this transaction states that the buffer holds only zeros now
  void declare_zero(TxnId txn, NodeId node) {
    Buf &b = buf();
    if (!b.buffer || !b.has_txn || !(b.txn == txn.raw_id()) || !b.writers.count(node.raw_id()))
      throw HazardError("declare_zero by a node that is not a writer of this transaction");
    b.all_zero = true;
  }
  // Marks the value to be carried into `txn` by the first read there (op.hh:236-247); a write in
  // the new transaction replaces it as usual.
  void rollover(TxnId txn) {
    Buf &b = buf();
    if (!(b.has_txn && b.txn == txn.raw_id())) b.rollover = true;
  }
  // Read access: the value must have been written in this transaction, or carried into it.
  V &get(TxnId txn, NodeId node) {
    Buf &b = buf();
    if (b.buffer && b.rollover && !(b.has_txn && b.txn == txn.raw_id())) {
      b.has_txn = true;
      b.txn = txn.raw_id();
      b.writers.clear();
      b.readers.clear();
      b.rollover = false;
    }
    if (!b.buffer || !b.has_txn || !(b.txn == txn.raw_id())) throw HazardError("read of a variable not written in this transaction");
    b.readers.insert(node.raw_id());
    return *b.buffer;
  }
  V &get_mut(TxnId txn, NodeId node) {
    Buf &b = buf();
    if (!b.buffer || !b.has_txn || !(b.txn == txn.raw_id()) || !b.writers.count(node.raw_id()))
      throw HazardError("get_mut by a node that is not a writer of this transaction");
    b.all_zero = false;
    return *b.buffer;
  }
  V &get_excl(TxnId txn, NodeId node) {
    V &v = get_mut(txn, node);
    if (buf().writers.size() != 1) throw HazardError("get_excl with more than one writer");
    return v;
  }
  bool written(TxnId txn) const { return buf().has_txn && buf().txn == txn.raw_id() && !buf().writers.empty(); }

private:
  struct Buf {
    VarId var;
    bool has_txn = false, rollover = false, all_zero = false;
    uint64_t txn = 0;
    std::set<uint64_t> writers, readers;
    std::unique_ptr<V> buffer;
    shared_ptr<Buf> forward;  // set: this variable is that one (forward_to)
  };
  shared_ptr<Buf> root() const {
    shared_ptr<Buf> b = buf_;
    while (b->forward) b = b->forward;
    return b;
  }
  Buf &buf() const {
    Buf *b = buf_.get();
    while (b->forward) b = b->forward.get();
    return *b;
  }
  bool begin(TxnId txn, Ctx *ctx) {
    Buf &b = buf();
    if (b.has_txn && b.txn == txn.raw_id()) return false;
    b.has_txn = true;
    b.txn = txn.raw_id();
    b.rollover = false;
    b.writers.clear();
    b.readers.clear();
    if (!b.buffer) allocate(ctx);
    return true;
  }
  void allocate(Ctx *ctx) {
    if constexpr (IsBatchArray<V>::value)
      buf().buffer.reset(new V(V::ZerosPadded(shape_, offset_, stride_, batch_shape_, ctx)));
    else
      buf().buffer.reset(new V(V::Zeros(shape_, ctx)));
    buf().all_zero = true;
  }
  VShape shape_, offset_, stride_;
  size_t batch_shape_ = 0;
  shared_ptr<Buf> buf_;
};

template <typename V>
class VarData {
public:
  typedef typename V::Shape VShape;
  VarData() {}
  explicit VarData(VShape shape, size_t batch_shape = 0) : val_(shape, batch_shape), grad_(shape, batch_shape) {}
  VarData(VShape shape, VShape offset, VShape stride, size_t batch_shape)
      : val_(shape, offset, stride, batch_shape), grad_(shape, offset, stride, batch_shape) {}
  VarData clone() const { return *this; }
  // Not in the reference.  This variable's gradient becomes the SAME buffer as `other`'s (same shape): whoever
  // writes one writes the other.  For a node whose input gradient equals its output gradient (a sum's) and whose
  // input has no other consumer: no copy is needed.
  void alias_grad(VarData &other) {
    if (other.shape() != shape() || other.offset() != offset() || other.stride() != stride() || other.batch_shape() != batch_shape())
      throw std::invalid_argument("VarData::alias_grad: the two variables must have one layout");
    grad_ = other.grad_;
  }
  // Not in the reference.  `other`'s gradient, in every copy of `other` that a node already holds, becomes this
  // variable's gradient buffer.
  void absorb_grad(VarData &other) { other.grad_.forward_to(grad_); }
  TxnVar<V> &val() { return val_; }
  TxnVar<V> &grad() { return grad_; }
  VShape shape() const { return val_.shape(); }
  VShape offset() const { return val_.offset(); }
  VShape stride() const { return val_.stride(); }
  size_t batch_shape() const { return val_.batch_shape(); }
  // op.hh:569-581
  void rollover_all(TxnId txn, VarIdSet &vars) {
    if (vars.contains(val_.var())) val_.rollover(txn);
    if (vars.contains(grad_.var())) grad_.rollover(txn);
  }

private:
  TxnVar<V> val_, grad_;
};

// ---------------------------------------------------------------------------
// traversal
// ---------------------------------------------------------------------------
// Counts visits per epoch so that a node with several consumers runs once on the way in
// (first push) and once on the way out (when every consumer has popped), op.hh:593-668.
class OperatorStack {
public:
  size_t push(EpochId e) { return sync(e), ++pushes_; }
  size_t degree(EpochId e) { return sync(e), pushes_; }
  size_t pop(EpochId e) { return sync(e), ++pops_; }

private:
  void sync(EpochId e) {
    if (!has_ || !(epoch_ == e.raw_id())) {
      has_ = true;
      epoch_ = e.raw_id();
      pushes_ = pops_ = 0;
    }
  }
  bool has_ = false;
  uint64_t epoch_ = 0;
  size_t pushes_ = 0, pops_ = 0;
};

// The arrays one walk over the graph contributes to (or takes from) a flat vector, in walk order.
// The reference copies array by array as the walk proceeds (store_any / load_any through an `any`
// reader or writer, op.hh:831-861); here the walk only collects and ONE batched copy follows it.
struct FlatBatch {
  vector<float *> arrays;
  vector<uint64_t> lens;
  hipStream_t stream = nullptr;
  size_t push(float *dptr, size_t len, hipStream_t s) {
    arrays.push_back(dptr);
    lens.push_back(len);
    stream = s;
    return len;
  }
};

class Op {
public:
  Op() {}
  virtual ~Op() {}
  NodeId id() const { return node_id_; }

  virtual void _push(EpochId epoch, function<void(Op *)> apply) = 0;
  virtual void _pop(EpochId epoch, function<void(Op *)> apply) = 0;
  virtual void _forward(TxnId txn) = 0;
  virtual void _backward(TxnId txn) = 0;
  virtual void _set_grad_sink(TxnId txn) { (void)txn; }
  // Flat-vector plumbing (op.hh:630-658): a node that owns variables of `vars` adds them to the
  // batch at the running offset and returns the advanced offset.  batch == NULL only measures.
  virtual size_t _load_val(TxnId, VarIdSet &, size_t offset, FlatBatch *) { return offset; }
  virtual size_t _load_grad(TxnId, VarIdSet &, size_t offset, FlatBatch *) { return offset; }
  virtual size_t _store_val(TxnId, VarIdSet &, size_t offset, FlatBatch *) { return offset; }
  virtual size_t _store_grad(TxnId, VarIdSet &, size_t offset, FlatBatch *) { return offset; }
  // Only nodes that own long-lived variables (parameters, statistics, inputs) carry anything over.
  virtual void _persist(TxnId, VarIdSet &) {}
  // Only parameters with an initialiser do anything (op.hh:654-656).
  virtual void _init(TxnId, std::mt19937_64 *) {}
  // Not in the reference, which always computes every input gradient.  false: nothing below this
  // node has parameters, so consumers need not produce (and this node's backward will not read)
  // the gradient of its output; the first layer's input gradient is the case that matters.
  virtual bool _requires_grad() { return true; }

  // The members of `vars` reachable from this node, in the order the backward walk meets them, as
  // consecutive ranges of a flat device vector starting at `offset`; returns the end offset
  // (src/op.cc:148-194).  store_* with a NULL writer only measures.  One batched copy per call,
  // enqueued on the stream of the variables' context.
  size_t load_val(TxnId txn, VarIdSet &vars, size_t offset, GPUMemory<float> *reader);
  size_t load_grad(TxnId txn, VarIdSet &vars, size_t offset, GPUMemory<float> *reader);
  size_t store_val(TxnId txn, VarIdSet &vars, size_t offset, GPUMemory<float> *writer);
  size_t store_grad(TxnId txn, VarIdSet &vars, size_t offset, GPUMemory<float> *writer);
  // marks the members of `vars` to keep their value into transaction `txn` (src/op.cc:205-212)
  void persist(TxnId txn, VarIdSet &vars);
  // gives every parameter below this node its initial value, in walk order (src/op.cc:196-203)
  void init(TxnId txn, std::mt19937_64 *rng);

  // forward pass of everything this node depends on, in dependency order (op.cc:196-221)
  void eval(TxnId txn) {
    EpochId e;
    _push(e, [txn](Op *op) { op->_forward(txn); });
    _pop(e, [](Op *) {});
  }
  // forward, seed this node's gradient, then backward in reverse order (op.cc:223-234)
  void gradient(TxnId txn) {
    EpochId e;
    _push(e, [txn](Op *op) { op->_forward(txn); });
    _set_grad_sink(txn);
    _pop(e, [txn](Op *op) { op->_backward(txn); });
  }

protected:
  OperatorStack stack_;

private:
  NodeId node_id_;
};

template <typename V>
class Var : public virtual Op {
public:
  virtual ~Var() {}
  virtual typename V::Shape shape() = 0;
  virtual typename V::Shape offset() = 0;
  virtual typename V::Shape stride() = 0;
  virtual size_t batch_shape() = 0;
  virtual VarData<V> data() = 0;
  virtual vector<VarId> vars() {
    VarData<V> d = data();
    return {d.val().var(), d.grad().var()};
  }
};

// boilerplate shared by ops that own one output VarData `y_`
#define ARRAYDIFF_VAR_ACCESSORS(V)                                   \
  virtual typename V::Shape shape() { return y_.shape(); }           \
  virtual typename V::Shape offset() { return y_.offset(); }         \
  virtual typename V::Shape stride() { return y_.stride(); }         \
  virtual size_t batch_shape() { return y_.batch_shape(); }          \
  virtual VarData<V> data() { return y_.clone(); }

inline GPUContext *gpu_ctx_of(const shared_ptr<Context> &ctx) {
  GPUContext *c = dynamic_cast<GPUContext *>(ctx.get());
  if (!c) throw std::invalid_argument("operator needs a GPUContext");
  return c;
}
inline MultiGPUContext *mgpu_ctx_of(const shared_ptr<Context> &ctx) {
  MultiGPUContext *c = dynamic_cast<MultiGPUContext *>(ctx.get());
  if (!c) throw std::invalid_argument("operator needs a MultiGPUContext");
  return c;
}

// ---------------------------------------------------------------------------
// sources
// ---------------------------------------------------------------------------
// A batch-array input fed from host memory (the role of the reference's SrcOp / IOOp,
// op.hh:699-1087, reduced to what the path's tests and tools need).
template <typename V>
class SrcOp : public virtual Op, public virtual Var<V> {
public:
  static shared_ptr<SrcOp<V>> Make(typename V::Shape shape, size_t batch_shape, shared_ptr<Context> ctx) {
    return make_shared<SrcOp<V>>(shape, batch_shape, ctx);
  }
  SrcOp(typename V::Shape shape, size_t batch_shape, shared_ptr<Context> ctx) : ctx_(ctx), y_(shape, batch_shape) {}

  // dense host data of shape (shape, batch_shape), copied in synchronously
  template <typename T>
  void load(TxnId txn, const T *host) {
    GPUContext *c = gpu_ctx_of(ctx_);
    if (y_.val().overwrite(txn, id(), c)) {
      GPUConn conn = c->conn();
      y_.val().get_excl(txn, id()).load_sync(host, conn);
    }
  }
  template <typename T>
  void store_grad(TxnId txn, T *host) {
    GPUConn conn = gpu_ctx_of(ctx_)->conn();
    y_.grad().get(txn, id()).store_sync(host, conn);
  }
  virtual void _push(EpochId e, function<void(Op *)> apply) {
    if (1 == stack_.push(e)) apply(this);
  }
  virtual void _pop(EpochId e, function<void(Op *)> apply) {
    if (stack_.degree(e) == stack_.pop(e)) apply(this);
  }
  virtual void _forward(TxnId) {}
  virtual void _backward(TxnId) {}
  virtual void _persist(TxnId txn, VarIdSet &vars) { y_.rollover_all(txn, vars); }
  // an input's gradient is computed (the reference's behaviour) unless the caller declines it
  void set_requires_grad(bool r) { requires_grad_ = r; }
  virtual bool _requires_grad() { return requires_grad_; }
  ARRAYDIFF_VAR_ACCESSORS(V)

private:
  shared_ptr<Context> ctx_;
  VarData<V> y_;
  bool requires_grad_ = true;
};

// A parameter (dense, no batch dimension), e.g. the conv filter GPUArray4D<float>.
template <typename A>
class ParamOp : public virtual Op, public virtual Var<A> {
public:
  static shared_ptr<ParamOp<A>> Make(typename A::Shape shape, shared_ptr<Context> ctx) {
    return make_shared<ParamOp<A>>(shape, ctx);
  }
  ParamOp(typename A::Shape shape, shared_ptr<Context> ctx) : ctx_(ctx), y_(shape) {}
  // The reference wraps a parameter in an InitOp (op.hh:1002-1060); here the parameter keeps its
  // own initialiser, run by Op::init.
  typedef function<void(A *, std::mt19937_64 *, shared_ptr<Context>)> InitFn;
  static shared_ptr<ParamOp<A>> Make(typename A::Shape shape, InitFn init_fn, shared_ptr<Context> ctx) {
    auto p = make_shared<ParamOp<A>>(shape, ctx);
    p->init_fn_ = init_fn;
    return p;
  }
  void set_init(InitFn init_fn) { init_fn_ = init_fn; }
  virtual void _init(TxnId txn, std::mt19937_64 *rng) {
    if (!init_fn_) return;
    if (y_.val().overwrite(txn, id(), gpu_ctx_of(ctx_))) init_fn_(&y_.val().get_excl(txn, id()), rng, ctx_);
  }
  template <typename T>
  void load(TxnId txn, const T *host) {
    GPUContext *c = gpu_ctx_of(ctx_);
    if (y_.val().overwrite(txn, id(), c)) {
      GPUConn conn = c->conn();
      y_.val().get_excl(txn, id()).load_sync(host, conn);
    }
  }
  template <typename T>
  void store_grad(TxnId txn, T *host) {
    GPUConn conn = gpu_ctx_of(ctx_)->conn();
    y_.grad().get(txn, id()).store_sync(host, conn);
  }
  // the value as transaction txn sees it, copied out synchronously
  template <typename T>
  void store(TxnId txn, T *host) {
    GPUConn conn = gpu_ctx_of(ctx_)->conn();
    y_.val().get(txn, id()).store_sync(host, conn);
  }
  virtual void _push(EpochId e, function<void(Op *)> apply) {
    if (1 == stack_.push(e)) apply(this);
  }
  virtual void _pop(EpochId e, function<void(Op *)> apply) {
    if (stack_.degree(e) == stack_.pop(e)) apply(this);
  }
  virtual void _forward(TxnId) {}
  virtual void _backward(TxnId) {}
  virtual void _persist(TxnId txn, VarIdSet &vars) { y_.rollover_all(txn, vars); }
  // the value (gradient) is replaced from the flat vector: this node becomes its writer (op.hh:831-847)
  virtual size_t _load_val(TxnId txn, VarIdSet &vars, size_t offset, FlatBatch *batch) {
    return vars.mask(y_.val().var()) ? offset + flat_in(y_.val(), txn, batch) : offset;
  }
  virtual size_t _load_grad(TxnId txn, VarIdSet &vars, size_t offset, FlatBatch *batch) {
    return vars.mask(y_.grad().var()) ? offset + flat_in(y_.grad(), txn, batch) : offset;
  }
  virtual size_t _store_val(TxnId txn, VarIdSet &vars, size_t offset, FlatBatch *batch) {
    return vars.mask(y_.val().var()) ? offset + flat_out(y_.val(), txn, batch) : offset;
  }
  virtual size_t _store_grad(TxnId txn, VarIdSet &vars, size_t offset, FlatBatch *batch) {
    return vars.mask(y_.grad().var()) ? offset + flat_out(y_.grad(), txn, batch) : offset;
  }
  virtual typename A::Shape shape() { return y_.shape(); }
  virtual typename A::Shape offset() { return y_.offset(); }
  virtual typename A::Shape stride() { return y_.stride(); }
  virtual size_t batch_shape() { return 0; }
  virtual VarData<A> data() { return y_.clone(); }

private:
  size_t flat_in(TxnVar<A> &v, TxnId txn, FlatBatch *batch) {
    GPUContext *c = gpu_ctx_of(ctx_);
    if (!v.overwrite(txn, id(), c)) throw HazardError("load of a variable another node wrote in this transaction");
    A &a = v.get_excl(txn, id());
    if (!a.is_packed()) throw std::invalid_argument("flat vectors hold packed arrays only");
    return batch->push(reinterpret_cast<float *>(a.dptr()), a.dim().flat_size(), c->conn().stream());
  }
  size_t flat_out(TxnVar<A> &v, TxnId txn, FlatBatch *batch) {
    if (!batch) return y_.shape().flat_size();
    A &a = v.get(txn, id());
    if (!a.is_packed()) throw std::invalid_argument("flat vectors hold packed arrays only");
    return batch->push(reinterpret_cast<float *>(a.dptr()), a.dim().flat_size(), gpu_ctx_of(ctx_)->conn().stream());
  }
  shared_ptr<Context> ctx_;
  VarData<A> y_;
  InitFn init_fn_;
};

// Initialisers (src/op.cc:286-408): a constant, Xavier's uniform(+-sqrt(6/(fanin+fanout))) and
// Kaiming's normal(0, sqrt(2/fanin)), drawn on the host in array order and copied in.
template <typename A>
typename ParamOp<A>::InitFn constant_init_gen(float c) {
  return [c](A *val, std::mt19937_64 *, shared_ptr<Context> ctx) {
    vector<float> buf(val->dim().flat_size(), c);
    GPUConn conn = gpu_ctx_of(ctx)->conn();
    val->load_sync(buf.data(), conn);
  };
}
template <typename A>
typename ParamOp<A>::InitFn zeros_init_gen() { return constant_init_gen<A>(0.0f); }
template <typename A>
typename ParamOp<A>::InitFn ones_init_gen() { return constant_init_gen<A>(1.0f); }
template <typename A>
typename ParamOp<A>::InitFn xavier_init_gen(size_t fanin, size_t fanout) {
  return [fanin, fanout](A *val, std::mt19937_64 *rng, shared_ptr<Context> ctx) {
    const float half_width = std::sqrt(6.0f / (float)(fanin + fanout));
    std::uniform_real_distribution<float> dist(-half_width, half_width);
    vector<float> buf(val->dim().flat_size());
    for (float &v : buf) v = dist(*rng);
    GPUConn conn = gpu_ctx_of(ctx)->conn();
    val->load_sync(buf.data(), conn);
  };
}
template <typename A>
typename ParamOp<A>::InitFn kaiming_init_gen(size_t fanin, size_t fanout) {
  (void)fanout;
  return [fanin](A *val, std::mt19937_64 *rng, shared_ptr<Context> ctx) {
    std::normal_distribution<float> dist(0.0f, std::sqrt(2.0f / (float)fanin));
    vector<float> buf(val->dim().flat_size());
    for (float &v : buf) v = dist(*rng);
    GPUConn conn = gpu_ctx_of(ctx)->conn();
    val->load_sync(buf.data(), conn);
  };
}

// A variable that is a view of another op's data (outputs of HaloExch2DOp, op.hh:2653-2659).
template <typename V>
class NoOp : public virtual Op, public virtual Var<V> {
public:
  NoOp(shared_ptr<Op> op, VarData<V> y) : op_(op), y_(y) {}
  virtual void _push(EpochId e, function<void(Op *)> apply) {
    if (1 == stack_.push(e)) op_->_push(e, apply);
  }
  virtual void _pop(EpochId e, function<void(Op *)> apply) {
    if (stack_.degree(e) == stack_.pop(e)) op_->_pop(e, apply);
  }
  virtual void _forward(TxnId) {}
  virtual void _backward(TxnId) {}
  virtual bool _requires_grad() { return op_->_requires_grad(); }
  ARRAYDIFF_VAR_ACCESSORS(V)

private:
  shared_ptr<Op> op_;
  VarData<V> y_;
};

// Test / tool sink: identity on the value, seeds the input's gradient from host memory.
template <typename V>
class HostGradSinkOp : public virtual Op, public virtual Var<V> {
public:
  static shared_ptr<HostGradSinkOp<V>> Make(shared_ptr<Var<V>> input, shared_ptr<Context> ctx) {
    return make_shared<HostGradSinkOp<V>>(input, ctx);
  }
  HostGradSinkOp(shared_ptr<Var<V>> input, shared_ptr<Context> ctx) : ctx_(ctx), input_(input), y_(input->data()) {}
  void set_host_grad(const float *g) { host_grad_ = g; }
  template <typename T>
  void store_val(TxnId txn, T *host) {
    GPUConn conn = gpu_ctx_of(ctx_)->conn();
    y_.val().get(txn, id()).store_sync(host, conn);
  }
  virtual void _push(EpochId e, function<void(Op *)> apply) {
    if (1 == stack_.push(e)) {
      input_->_push(e, apply);
      apply(this);
    }
  }
  virtual void _pop(EpochId e, function<void(Op *)> apply) {
    if (stack_.degree(e) == stack_.pop(e)) {
      apply(this);
      input_->_pop(e, apply);
    }
  }
  virtual void _forward(TxnId) {}
  virtual void _backward(TxnId) {}
  virtual void _set_grad_sink(TxnId txn) {
    GPUContext *c = gpu_ctx_of(ctx_);
    const float *g = host_grad_;
    y_.grad().accumulate(txn, id(), c, [c, g](V *grad) {
      GPUConn conn = c->conn();
      grad->load_sync(g, conn);
    });
  }
  ARRAYDIFF_VAR_ACCESSORS(V)

private:
  shared_ptr<Context> ctx_;
  shared_ptr<Var<V>> input_;
  VarData<V> y_;
  const float *host_grad_ = nullptr;
};

// ---------------------------------------------------------------------------
// single-input ops share their traversal
// ---------------------------------------------------------------------------
template <typename V>
class UnaryVarOp : public virtual Op, public virtual Var<V> {
public:
  UnaryVarOp(shared_ptr<Var<V>> input, shared_ptr<Context> ctx) : ctx_(ctx), input_(input), x_(input->data()) {}
  virtual void _push(EpochId e, function<void(Op *)> apply) {
    if (1 == stack_.push(e)) {
      input_->_push(e, apply);
      apply(this);
    }
  }
  virtual void _pop(EpochId e, function<void(Op *)> apply) {
    if (stack_.degree(e) == stack_.pop(e)) {
      apply(this);
      input_->_pop(e, apply);
    }
  }
  // single-input ops have no parameters of their own
  virtual bool _requires_grad() { return input_->_requires_grad(); }
  ARRAYDIFF_VAR_ACCESSORS(V)

protected:
  shared_ptr<Context> ctx_;
  shared_ptr<Var<V>> input_;
  VarData<V> x_;
  VarData<V> y_;
};

template <typename V>
static vector<shared_ptr<Var<V>>> make_per_rank(
    shared_ptr<Context> ctx, function<shared_ptr<Var<V>>(size_t rank, shared_ptr<Context> dev_ctx)> make) {
  MultiGPUContext *m = mgpu_ctx_of(ctx);
  vector<shared_ptr<Var<V>>> out;
  for (size_t r = 0; r < m->num_ranks(); ++r) out.push_back(make(r, m->device_context(r)));
  return out;
}

// SpatialScatter2DOp: rows [rank*H/K, (rank+1)*H/K) of the full input -> this rank's tile.
template <typename V>
class SpatialScatter2DOp : public UnaryVarOp<V> {
public:
  static shared_ptr<Var<V>> Make(size_t rank, size_t num_ranks, shared_ptr<Var<V>> input, shared_ptr<Context> ctx) {
    return make_shared<SpatialScatter2DOp<V>>(rank, num_ranks, input, ctx);
  }
  // inputs.at(rank) is the (replicated) full tensor seen by that rank
  static vector<shared_ptr<Var<V>>> MakeParallel(vector<shared_ptr<Var<V>>> inputs, shared_ptr<Context> ctx) {
    const size_t k = mgpu_ctx_of(ctx)->num_ranks();
    return make_per_rank<V>(ctx, [&](size_t r, shared_ptr<Context> dc) { return Make(r, k, inputs.at(r), dc); });
  }
  SpatialScatter2DOp(size_t rank, size_t num_ranks, shared_ptr<Var<V>> input, shared_ptr<Context> ctx)
      : UnaryVarOp<V>(input, ctx), rank_(rank), num_ranks_(num_ranks) {
    this->y_ = VarData<V>(_get_output_shape(input->shape()), input->batch_shape());
  }
  typename V::Shape _get_output_shape(typename V::Shape in_shape) {
    if (in_shape.shape[1] % num_ranks_ != 0) throw std::invalid_argument("SpatialScatter2DOp: H % num_ranks != 0");
    return typename V::Shape(in_shape.shape[0], in_shape.shape[1] / num_ranks_, in_shape.shape[2]);
  }
  virtual void _forward(TxnId txn);
  virtual void _backward(TxnId txn);

private:
  size_t rank_, num_ranks_;
};

// SpatialGather2DOp: this rank's tile -> rows [rank*H/K, ...) of a zeroed full-size tensor.
// In the reference every rank produces a partially filled full tensor and an AllreduceOp sums
// them (src/zoo.cc:1841-1842); MakeJoined is the one-memory form: all ranks write their rows
// into ONE output.
template <typename V>
class SpatialGather2DOp : public UnaryVarOp<V> {
public:
  static shared_ptr<Var<V>> Make(size_t rank, size_t num_ranks, shared_ptr<Var<V>> input, shared_ptr<Context> ctx) {
    return make_shared<SpatialGather2DOp<V>>(rank, num_ranks, input, ctx);
  }
  static vector<shared_ptr<Var<V>>> MakeParallel(vector<shared_ptr<Var<V>>> inputs, shared_ptr<Context> ctx) {
    const size_t k = mgpu_ctx_of(ctx)->num_ranks();
    return make_per_rank<V>(ctx, [&](size_t r, shared_ptr<Context> dc) { return Make(r, k, inputs.at(r), dc); });
  }
  SpatialGather2DOp(size_t rank, size_t num_ranks, shared_ptr<Var<V>> input, shared_ptr<Context> ctx)
      : UnaryVarOp<V>(input, ctx), rank_(rank), num_ranks_(num_ranks) {
    auto s = input->shape();
    this->y_ = VarData<V>(typename V::Shape(s.shape[0], s.shape[1] * num_ranks, s.shape[2]), input->batch_shape());
  }
  virtual void _forward(TxnId txn);
  virtual void _backward(TxnId txn);

private:
  size_t rank_, num_ranks_;
};

// The one-memory form of gather: K unpadded tiles -> ONE full tensor in a single launch (an
// all-gather along H); backward hands each rank its rows of the gradient.
template <typename V>
class SpatialJoinedGather2DOp : public virtual Op, public virtual Var<V> {
public:
  static shared_ptr<SpatialJoinedGather2DOp<V>> Make(vector<shared_ptr<Var<V>>> inputs, shared_ptr<Context> ctx) {
    return make_shared<SpatialJoinedGather2DOp<V>>(inputs, ctx);
  }
  SpatialJoinedGather2DOp(vector<shared_ptr<Var<V>>> inputs, shared_ptr<Context> ctx) : ctx_(ctx), inputs_(inputs) {
    if (inputs.empty() || inputs.size() > ADH_MAX_TILES) throw std::invalid_argument("SpatialJoinedGather2DOp: 1..16 tiles");
    for (auto &in : inputs) {
      if (in->shape() != inputs[0]->shape()) throw std::invalid_argument("SpatialJoinedGather2DOp: tile shapes differ");
      xs_.push_back(in->data());
    }
    auto s = inputs[0]->shape();
    y_ = VarData<V>(typename V::Shape(s.shape[0], s.shape[1] * inputs.size(), s.shape[2]), inputs[0]->batch_shape());
  }
  template <typename T>
  void store_val(TxnId txn, T *host) {
    GPUConn conn = mgpu_ctx_of(ctx_)->device_context(0)->conn();
    y_.val().get(txn, id()).store_sync(host, conn);
  }
  virtual void _push(EpochId e, function<void(Op *)> apply) {
    if (1 == stack_.push(e)) {
      for (auto &in : inputs_) in->_push(e, apply);
      apply(this);
    }
  }
  virtual void _pop(EpochId e, function<void(Op *)> apply) {
    if (stack_.degree(e) == stack_.pop(e)) {
      apply(this);
      for (size_t r = inputs_.size(); r-- > 0;) inputs_.at(r)->_pop(e, apply);
    }
  }
  virtual void _forward(TxnId txn);
  virtual void _backward(TxnId txn);
  ARRAYDIFF_VAR_ACCESSORS(V)

private:
  shared_ptr<Context> ctx_;
  vector<shared_ptr<Var<V>>> inputs_;
  vector<VarData<V>> xs_;
  VarData<V> y_;
};

template <typename V>
class HaloPad2DOp : public UnaryVarOp<V> {
public:
  static shared_ptr<Var<V>> Make(size_t halo_pad, shared_ptr<Var<V>> input, shared_ptr<Context> ctx) {
    return make_shared<HaloPad2DOp<V>>(halo_pad, input, ctx);
  }
  static vector<shared_ptr<Var<V>>> MakeParallel(size_t halo_pad, vector<shared_ptr<Var<V>>> inputs,
                                                 shared_ptr<Context> ctx) {
    return make_per_rank<V>(ctx, [&](size_t r, shared_ptr<Context> dc) { return Make(halo_pad, inputs.at(r), dc); });
  }
  HaloPad2DOp(size_t halo_pad, shared_ptr<Var<V>> input, shared_ptr<Context> ctx)
      : UnaryVarOp<V>(input, ctx), halo_pad_(halo_pad) {
    this->y_ = VarData<V>(input->shape(), _get_output_offset(input->shape()), _get_output_stride(input->shape()),
                          input->batch_shape());
  }
  typename V::Shape _get_output_offset(typename V::Shape) { return typename V::Shape(halo_pad_, halo_pad_, 0); }
  typename V::Shape _get_output_stride(typename V::Shape s) {
    return typename V::Shape(s.shape[0] + 2 * halo_pad_, s.shape[1] + 2 * halo_pad_, s.shape[2]).packed_stride();
  }
  virtual void _forward(TxnId txn);
  virtual void _backward(TxnId txn);

private:
  size_t halo_pad_;
};

template <typename V>
class HaloUnpad2DOp : public UnaryVarOp<V> {
public:
  static shared_ptr<Var<V>> Make(size_t halo_pad, shared_ptr<Var<V>> input, shared_ptr<Context> ctx) {
    return make_shared<HaloUnpad2DOp<V>>(halo_pad, input, ctx);
  }
  static vector<shared_ptr<Var<V>>> MakeParallel(size_t halo_pad, vector<shared_ptr<Var<V>>> inputs,
                                                 shared_ptr<Context> ctx) {
    return make_per_rank<V>(ctx, [&](size_t r, shared_ptr<Context> dc) { return Make(halo_pad, inputs.at(r), dc); });
  }
  HaloUnpad2DOp(size_t halo_pad, shared_ptr<Var<V>> input, shared_ptr<Context> ctx)
      : UnaryVarOp<V>(input, ctx), halo_pad_(halo_pad) {
    this->y_ = VarData<V>(input->shape(), input->batch_shape());
  }
  virtual void _forward(TxnId txn);
  virtual void _backward(TxnId txn);

private:
  size_t halo_pad_;
};

template <typename V>
class HaloRepad2DOp : public UnaryVarOp<V> {
public:
  static shared_ptr<Var<V>> Make(size_t src_halo_pad, size_t dst_halo_pad, shared_ptr<Var<V>> input,
                                 shared_ptr<Context> ctx) {
    return make_shared<HaloRepad2DOp<V>>(src_halo_pad, dst_halo_pad, input, ctx);
  }
  static vector<shared_ptr<Var<V>>> MakeParallel(size_t src_halo_pad, size_t dst_halo_pad,
                                                 vector<shared_ptr<Var<V>>> inputs, shared_ptr<Context> ctx) {
    return make_per_rank<V>(
        ctx, [&](size_t r, shared_ptr<Context> dc) { return Make(src_halo_pad, dst_halo_pad, inputs.at(r), dc); });
  }
  HaloRepad2DOp(size_t src_halo_pad, size_t dst_halo_pad, shared_ptr<Var<V>> input, shared_ptr<Context> ctx)
      : UnaryVarOp<V>(input, ctx), src_pad_(src_halo_pad), dst_pad_(dst_halo_pad) {
    auto s = input->shape();
    this->y_ = VarData<V>(s, typename V::Shape(dst_pad_, dst_pad_, 0),
                          typename V::Shape(s.shape[0] + 2 * dst_pad_, s.shape[1] + 2 * dst_pad_, s.shape[2]).packed_stride(),
                          input->batch_shape());
  }
  virtual void _forward(TxnId txn);
  // the reference defines no backward for this op (src/op.cc:2872-2960 holds the forward only)
  virtual void _backward(TxnId) { throw std::logic_error("HaloRepad2DOp has no backward"); }

private:
  size_t src_pad_, dst_pad_;
};

// One node spanning all ranks, in place on the K pad outputs; the outputs are NoOp views of
// the same VarData.
template <typename V>
class HaloExch2DOp : public virtual Op {
public:
  // forward_by_consumer (not in the reference): neither pass launches anything, because the consumer is a
  // convolution built with Conv2DShape::unexchanged_rows: its forward pass reads the neighbours' rows itself
  // and its input gradient arrives reduced (the neighbours' gradient rows are multiplied by the tile that
  // owns the result).
  static vector<shared_ptr<Var<V>>> MakeParallel(size_t halo_pad, vector<shared_ptr<Var<V>>> inputs,
                                                 shared_ptr<Context> ctx, bool forward_by_consumer = false) {
    auto op = make_shared<HaloExch2DOp<V>>(halo_pad, inputs, ctx, forward_by_consumer);
    vector<shared_ptr<Var<V>>> outputs;
    for (size_t r = 0; r < inputs.size(); ++r) outputs.push_back(make_shared<NoOp<V>>(op, op->xs_.at(r).clone()));
    return outputs;
  }
  HaloExch2DOp(size_t halo_pad, vector<shared_ptr<Var<V>>> inputs, shared_ptr<Context> ctx,
               bool forward_by_consumer = false)
      : ctx_(ctx), halo_pad_(halo_pad), forward_by_consumer_(forward_by_consumer), inputs_(inputs) {
    if (inputs.size() != mgpu_ctx_of(ctx)->num_ranks()) throw std::invalid_argument("HaloExch2DOp: one input per rank");
    for (auto &in : inputs) xs_.push_back(in->data());
  }
  virtual void _push(EpochId e, function<void(Op *)> apply) {
    if (1 == stack_.push(e)) {
      for (auto &in : inputs_) in->_push(e, apply);
      apply(this);
    }
  }
  virtual void _pop(EpochId e, function<void(Op *)> apply) {
    if (stack_.degree(e) == stack_.pop(e)) {
      apply(this);
      for (size_t r = inputs_.size(); r-- > 0;) inputs_.at(r)->_pop(e, apply);
    }
  }
  virtual bool _requires_grad() {
    for (auto &in : inputs_)
      if (in->_requires_grad()) return true;
    return false;
  }
  virtual void _forward(TxnId txn);
  virtual void _backward(TxnId txn);

private:
  shared_ptr<Context> ctx_;
  size_t halo_pad_;
  bool forward_by_consumer_;
  vector<shared_ptr<Var<V>>> inputs_;
  vector<VarData<V>> xs_;
};

// ---------------------------------------------------------------------------
// convolution over the halo-padded slab
// ---------------------------------------------------------------------------
class Conv2DShape {
public:
  size_t filters;
  array<size_t, 2> axes;
  array<size_t, 2> kernel;
  array<size_t, 2> dilate;
  array<size_t, 2> stride;
  array<size_t, 2> pad;
  bool halo_padded_input;
  bool enable_hmma;
  // Not in the reference.  A promise that the ranks' filter variables hold equal values (the
  // parallel optimizer keeps them so): all tiles are then convolved in ONE launch with rank 0's
  // filter, and the filter gradient of all tiles goes to rank 0's variable in one launch while
  // the other ranks' gradients are zero.  The sum over ranks, which is all the optimizer uses,
  // is the same.
  bool replicated_filters = false;
  // Not in the reference.  The inputs are the row tiles of one activation in rank order (a 1 x K grid)
  // whose inner halo rows nobody exchanged (HaloExch2DOp made with forward_by_consumer): the forward
  // pass and the filter gradient read those rows from the neighbouring tiles, or exchange them first
  // where the kernel for the shape cannot (or where the ranks' filters differ, so that one launch cannot
  // hold every tile); the input gradient comes out as after the halo reduce (by a kernel that reads the
  // neighbours' gradient rows, or by a reduce after the ordinary one).  The input gradient must have no
  // other contributor.
  bool unexchanged_rows = false;
  // Not in the reference.  The inputs are the row tiles of one activation in rank order (a 1 x K grid) and
  // carry NO halo (halo_padded_input = false; pad is the zero padding of the unsplit convolution): the op is
  // the reference's HaloPad2DOp -> HaloExch2DOp -> conv chain in one node.  Zero padding at the tensor's border
  // and the neighbours' rows at the tiles' borders are read by the kernels; the input gradient comes out
  // unpadded and complete.  Any window whose row split stitches: tile height a multiple of the row stride,
  // 0 < (kernel - 1) * dilation + 1 - 2 * pad <= stride along the rows, a window that reaches the adjacent
  // tiles only (3x3 pad 1 at stride 1 or 2, the 7x7 stem with pad 3, 1x1 pad 0 ...).
  bool unpadded_tiles = false;
};

// V = GPUBatchArray3D<float>, A = GPUArray4D<float> (filter, Shape4D(kw,kh,Cin,Cout) = KCRS).
// Any window / stride / dilation; an optional bias per output channel (GPUArray1D<float>, one variable per rank
// like the filter: y += bias after the conv, its gradient the sum of dy over images and pixels,
// src/op.cc:1602-1610, 1632-1648).  With halo_padded_input the input's halo must equal the
// conv pad (the padded tile is convolved with pad 0, src/op.cc:1392-1410); without it the input
// must be packed and pad must be 0 (the 1x1 projections, src/zoo.cc:680-690).  Implicit zero
// padding of an unpadded input is not part of this path and throws at construction.  3x3 /
// stride 1 / dilation 1 over halo 1 (the spatially-parallel blocks, src/zoo.cc:577-652) runs the
// kernels written for it, everything else the general ones.
// One node serves all ranks it was made for: the K slabs go to the device in ONE launch per
// pass (the reference ran one cuDNN call per rank on K GPUs).  Make() is the one-rank form and
// is itself the output variable; MakeParallel() returns per-rank views of one node.
template <typename V, typename A>
class SlabConv2DOp : public virtual Op, public virtual Var<V> {
public:
  typedef GPUArray1D<float> Bias;
  static shared_ptr<Var<V>> Make(Conv2DShape shape, shared_ptr<Var<V>> input, shared_ptr<Var<A>> kernel,
                                 shared_ptr<Context> ctx) {
    return make_shared<SlabConv2DOp<V, A>>(shape, vector<shared_ptr<Var<V>>>{input},
                                           vector<shared_ptr<Var<A>>>{kernel}, ctx);
  }
  // the reference's constructor with a bias (op.hh:1828-1850): (shape, input, kernel, bias, ctx)
  static shared_ptr<Var<V>> Make(Conv2DShape shape, shared_ptr<Var<V>> input, shared_ptr<Var<A>> kernel,
                                 shared_ptr<Var<Bias>> bias, shared_ptr<Context> ctx) {
    return make_shared<SlabConv2DOp<V, A>>(shape, vector<shared_ptr<Var<V>>>{input}, vector<shared_ptr<Var<A>>>{kernel},
                                           ctx, vector<shared_ptr<Var<V>>>{}, vector<shared_ptr<Var<Bias>>>{bias});
  }
  // each rank holds its own copy of the filter in the reference; here kernels.at(r) may all be
  // the same variable, its gradient then accumulates over the tiles
  // residuals (not in the reference; tiles without halo only): residuals.at(r) is added to rank r's result,
  // y = conv(x, w) + residual, the sum that closes a residual block, in the convolution's own stores where the 3x3
  // kernel serves the shape (else one pass that adds in place).  The residual's gradient is the output's gradient:
  // its variable forwards to the output's, so the backward pass does nothing for it.  As with JoinOp's trunk_input,
  // every other consumer of a residual must lie UPSTREAM of this node's input (the block input, whose other
  // consumer is the first node of the path that ends here) or the residual must have no other consumer (the
  // projection of a block that changes extents): those nodes then add to the shared buffer after this node has read it.
  // biases: empty, or one variable of `filters` numbers per rank (with replicated_filters the ranks' biases are
  // promised equal like their filters: rank 0's is added to every tile and receives every tile's gradient)
  static vector<shared_ptr<Var<V>>> MakeParallel(Conv2DShape shape, vector<shared_ptr<Var<V>>> inputs,
                                                 vector<shared_ptr<Var<A>>> kernels, shared_ptr<Context> ctx,
                                                 vector<shared_ptr<Var<V>>> residuals = {},
                                                 vector<shared_ptr<Var<Bias>>> biases = {}) {
    auto op = make_shared<SlabConv2DOp<V, A>>(shape, inputs, kernels, ctx, residuals, biases);
    vector<shared_ptr<Var<V>>> outputs;
    for (size_t r = 0; r < inputs.size(); ++r) outputs.push_back(make_shared<NoOp<V>>(op, op->ys_.at(r).clone()));
    return outputs;
  }
  SlabConv2DOp(Conv2DShape shape, vector<shared_ptr<Var<V>>> inputs, vector<shared_ptr<Var<A>>> kernels,
               shared_ptr<Context> ctx, vector<shared_ptr<Var<V>>> residuals = {},
               vector<shared_ptr<Var<Bias>>> biases = {})
      : ctx_(ctx), shape_(shape), x_vars_(inputs), kernel_vars_(kernels), res_vars_(residuals), bias_vars_(biases) {
    if (shape.kernel[0] == 0 || shape.kernel[1] == 0 || shape.stride[0] == 0 || shape.stride[1] == 0 ||
        shape.dilate[0] == 0 || shape.dilate[1] == 0)
      throw std::invalid_argument("SlabConv2DOp: empty window, stride or dilation");
    if (shape.unpadded_tiles) {
      const size_t span = (shape.kernel[1] - 1) * shape.dilate[1] + 1;
      const size_t tile_h = inputs.empty() ? 0 : inputs[0]->shape().shape[1];
      if (shape.halo_padded_input || 2 * shape.pad[1] >= span || span - 2 * shape.pad[1] > shape.stride[1] ||
          tile_h % shape.stride[1] != 0 || shape.pad[1] > tile_h || span - 1 - shape.pad[1] > tile_h)
        throw std::invalid_argument("SlabConv2DOp: tiles without halo need a row split whose outputs stitch");
    } else if (!shape.halo_padded_input && (shape.pad[0] != 0 || shape.pad[1] != 0))
      throw std::invalid_argument("SlabConv2DOp: padding needs a halo-padded input");
    if (inputs.empty() || inputs.size() != kernels.size() || inputs.size() > ADH_MAX_TILES)
      throw std::invalid_argument("SlabConv2DOp: one kernel variable per input");
    if (shape.unexchanged_rows && !(shape.halo_padded_input && shape.pad[0] == 1 && shape.pad[1] == 1))
      throw std::invalid_argument("SlabConv2DOp: unexchanged rows need a halo of one");
    for (size_t r = 0; r < inputs.size(); ++r) {
      auto off = inputs[r]->offset();
      const size_t halo0 = shape.unpadded_tiles ? 0 : shape.pad[0], halo1 = shape.unpadded_tiles ? 0 : shape.pad[1];
      if (off.shape[0] != halo0 || off.shape[1] != halo1 || off.shape[2] != 0)
        throw std::invalid_argument("SlabConv2DOp: input halo must equal the conv pad");
      if (inputs[r]->shape() != inputs[0]->shape() || inputs[r]->batch_shape() != inputs[0]->batch_shape())
        throw std::invalid_argument("SlabConv2DOp: all slabs must have one shape");
      xs_.push_back(inputs[r]->data());
      kernels_.push_back(kernels[r]->data());
      ys_.push_back(VarData<V>(_get_output_shape(inputs[r]->shape(), inputs[r]->batch_shape()), inputs[r]->batch_shape()));
    }
    if (!biases.empty()) {
      if (biases.size() != inputs.size()) throw std::invalid_argument("SlabConv2DOp: one bias variable per input");
      for (size_t r = 0; r < biases.size(); ++r) {
        if (biases[r]->shape() != Shape1D(shape.filters))
          throw std::invalid_argument("SlabConv2DOp: a bias holds one number per filter");
        biases_.push_back(biases[r]->data());
      }
    }
    if (!residuals.empty()) {
      if (!shape.unpadded_tiles || residuals.size() != inputs.size())
        throw std::invalid_argument("SlabConv2DOp: one residual per tile, over tiles without halo");
      for (size_t r = 0; r < residuals.size(); ++r) {
        if (residuals[r]->shape() != ys_[r].shape() || residuals[r]->batch_shape() != ys_[r].batch_shape() ||
            !residuals[r]->offset().is_zero())
          throw std::invalid_argument("SlabConv2DOp: a residual must be packed and of the output's shape");
        res_.push_back(residuals[r]->data());
        ys_[r].absorb_grad(res_[r]);
      }
    }
  }
  // out = floor((in + 2p - ((k-1)d+1)) / s) + 1 per axis (op.cc:1512-1523)
  Shape3D _get_output_shape(Shape3D in_shape, size_t) {
    size_t out[2];
    for (int a = 0; a < 2; ++a) {
      const size_t padded = in_shape.shape[a] + 2 * shape_.pad[a], span = (shape_.kernel[a] - 1) * shape_.dilate[a] + 1;
      if (padded < span) throw std::invalid_argument("SlabConv2DOp: window larger than the padded input");
      out[a] = (padded - span) / shape_.stride[a] + 1;
    }
    return Shape3D(out[0], out[1], shape_.filters);
  }
  bool is_3x3_unit_unpadded() const {
    return shape_.kernel[0] == 3 && shape_.kernel[1] == 3 && shape_.stride[0] == 1 && shape_.stride[1] == 1 &&
           shape_.dilate[0] == 1 && shape_.dilate[1] == 1 && shape_.pad[0] == 1 && shape_.pad[1] == 1 &&
           !shape_.halo_padded_input && shape_.unpadded_tiles;
  }
  bool is_3x3_unit() const {
    return shape_.kernel[0] == 3 && shape_.kernel[1] == 3 && shape_.stride[0] == 1 && shape_.stride[1] == 1 &&
           shape_.dilate[0] == 1 && shape_.dilate[1] == 1 && shape_.pad[0] == 1 && shape_.pad[1] == 1 &&
           shape_.halo_padded_input;
  }
  virtual void _push(EpochId e, function<void(Op *)> apply) {
    if (1 == stack_.push(e)) {
      for (auto &res : res_vars_) res->_push(e, apply);
      for (size_t r = 0; r < x_vars_.size(); ++r) {
        x_vars_[r]->_push(e, apply);
        kernel_vars_[r]->_push(e, apply);
        if (!bias_vars_.empty()) bias_vars_[r]->_push(e, apply);
      }
      apply(this);
    }
  }
  virtual void _pop(EpochId e, function<void(Op *)> apply) {
    if (stack_.degree(e) == stack_.pop(e)) {
      apply(this);
      for (size_t r = x_vars_.size(); r-- > 0;) {
        if (!bias_vars_.empty()) bias_vars_[r]->_pop(e, apply);
        kernel_vars_[r]->_pop(e, apply);
        x_vars_[r]->_pop(e, apply);
      }
      for (size_t r = res_vars_.size(); r-- > 0;) res_vars_[r]->_pop(e, apply);
    }
  }
  virtual void _forward(TxnId txn);
  virtual void _backward(TxnId txn);
  virtual typename V::Shape shape() { return ys_[0].shape(); }
  virtual typename V::Shape offset() { return ys_[0].offset(); }
  virtual typename V::Shape stride() { return ys_[0].stride(); }
  virtual size_t batch_shape() { return ys_[0].batch_shape(); }
  virtual VarData<V> data() { return ys_[0].clone(); }

private:
  shared_ptr<Context> ctx_;
  Conv2DShape shape_;
  vector<shared_ptr<Var<V>>> x_vars_;
  vector<shared_ptr<Var<A>>> kernel_vars_;
  vector<VarData<V>> xs_;
  vector<VarData<A>> kernels_;
  vector<VarData<V>> ys_;
  vector<shared_ptr<Var<V>>> res_vars_;  // empty, or one per tile: added to the result
  vector<VarData<V>> res_;
  vector<shared_ptr<Var<Bias>>> bias_vars_;  // empty, or one per rank
  vector<VarData<Bias>> biases_;
  void backward_bias(TxnId txn);
};
// the third parameter is the reference's bias array type; the bias here is always GPUArray1D<float>
template <typename V, typename A, typename B = A>
using CudnnConv2DOp = SlabConv2DOp<V, A>;

// ---------------------------------------------------------------------------
// the shard-local ops between two halo exchanges: batch norm, rectifier, sum join
// ---------------------------------------------------------------------------
template <typename V, typename B>
class BatchNormOutput {
public:
  shared_ptr<Var<V>> op;
  shared_ptr<Var<B>> batch_mean;
  shared_ptr<Var<B>> batch_variance;
  shared_ptr<Var<B>> fixed_mean;
  shared_ptr<Var<B>> fixed_variance;
  shared_ptr<Var<B>> scale;
  shared_ptr<Var<B>> shift;
  VarIdSet params;
  VarIdSet grads;
  VarIdSet batch_stats;
  VarIdSet fixed_stats;
};

// additions to the reference's struct: the per-rank parameter variables, so that a caller can load them
template <typename V, typename B>
class ParallelBatchNormOutput {
public:
  vector<shared_ptr<Var<V>>> ops;
  vector<VarIdSet> params;
  vector<VarIdSet> grads;
  vector<VarIdSet> batch_stats;
  vector<VarIdSet> fixed_stats;
  vector<shared_ptr<ParamOp<B>>> scales, shifts, fixed_means, fixed_variances, batch_means, batch_variances;
};

// Switch = bool, V = GPUBatchArray3D<float>, B = GPUArray1D<float>.  *switch_var == false: batch
// statistics of THIS rank's tile (training), true: the fixed statistics (evaluation; its backward
// is unimplemented in the reference too, src/op.cc:4078-4080).  One node serves all ranks it was
// made for (one launch per pass over all tiles); every rank keeps its own parameters and statistics.
// Unlike the reference's Make(), the parameters start uninitialised: load scale / shift (and the fixed
// statistics for evaluation) through the ParamOps in the output before the first transaction.
template <typename Switch, typename V, typename B>
class SlabBatchNorm2DOp : public virtual Op, public virtual Var<V> {
public:
  struct RankVars {
    shared_ptr<ParamOp<B>> batch_mean, batch_variance, fixed_mean, fixed_variance, scale, shift;
  };
  static RankVars make_rank_vars(size_t channels, shared_ptr<Context> dev_ctx) {
    RankVars v;
    typename B::Shape s(channels);
    // initial values as in the reference's Make (op.hh:3173-3211): used only if Op::init runs
    v.batch_mean = ParamOp<B>::Make(s, dev_ctx);
    v.batch_variance = ParamOp<B>::Make(s, dev_ctx);
    v.fixed_mean = ParamOp<B>::Make(s, zeros_init_gen<B>(), dev_ctx);
    v.fixed_variance = ParamOp<B>::Make(s, ones_init_gen<B>(), dev_ctx);
    v.scale = ParamOp<B>::Make(s, ones_init_gen<B>(), dev_ctx);
    v.shift = ParamOp<B>::Make(s, zeros_init_gen<B>(), dev_ctx);
    return v;
  }
  static BatchNormOutput<V, B> Make(size_t channels, shared_ptr<Switch> switch_var, shared_ptr<Var<V>> input,
                                    shared_ptr<Context> ctx) {
    RankVars v = make_rank_vars(channels, ctx);
    auto op = make_shared<SlabBatchNorm2DOp<Switch, V, B>>(switch_var, vector<shared_ptr<Var<V>>>{input},
                                                           vector<RankVars>{v}, ctx);
    BatchNormOutput<V, B> out;
    out.op = op;
    out.batch_mean = v.batch_mean; out.batch_variance = v.batch_variance;
    out.fixed_mean = v.fixed_mean; out.fixed_variance = v.fixed_variance;
    out.scale = v.scale; out.shift = v.shift;
    fill_sets(v, &out.params, &out.grads, &out.batch_stats, &out.fixed_stats);
    return out;
  }
  // relu / out_halo (not in the reference): the node also applies the rectifier and writes into the
  // interior of a tile padded by out_halo with a zeroed border, i.e. it stands for the chain
  // CudnnBatchNorm2DOp -> CudnnActivationOp -> HaloPad2DOp (src/zoo.cc:596-604) in ONE pass over the
  // data; its outputs then go straight to HaloExch2DOp.
  static ParallelBatchNormOutput<V, B> MakeParallel(size_t channels, shared_ptr<Switch> switch_var,
                                                    vector<shared_ptr<Var<V>>> inputs, shared_ptr<Context> ctx,
                                                    bool relu = false, size_t out_halo = 0) {
    MultiGPUContext *m = mgpu_ctx_of(ctx);
    vector<RankVars> vars;
    for (size_t r = 0; r < inputs.size(); ++r) vars.push_back(make_rank_vars(channels, m->device_context(r)));
    auto op = make_shared<SlabBatchNorm2DOp<Switch, V, B>>(switch_var, inputs, vars, ctx, relu, out_halo);
    ParallelBatchNormOutput<V, B> out;
    for (size_t r = 0; r < inputs.size(); ++r) {
      out.ops.push_back(make_shared<NoOp<V>>(op, op->ys_.at(r).clone()));
      VarIdSet p, g, bs, fs;
      fill_sets(vars[r], &p, &g, &bs, &fs);
      out.params.push_back(p); out.grads.push_back(g); out.batch_stats.push_back(bs); out.fixed_stats.push_back(fs);
      out.scales.push_back(vars[r].scale); out.shifts.push_back(vars[r].shift);
      out.fixed_means.push_back(vars[r].fixed_mean); out.fixed_variances.push_back(vars[r].fixed_variance);
      out.batch_means.push_back(vars[r].batch_mean); out.batch_variances.push_back(vars[r].batch_variance);
    }
    return out;
  }
  SlabBatchNorm2DOp(shared_ptr<Switch> switch_var, vector<shared_ptr<Var<V>>> inputs, vector<RankVars> vars,
                    shared_ptr<Context> ctx, bool relu = false, size_t out_halo = 0)
      : ctx_(ctx), switch_var_(switch_var), x_vars_(inputs), vars_(vars), relu_(relu), out_halo_(out_halo) {
    if (inputs.empty() || inputs.size() != vars.size() || inputs.size() > ADH_MAX_TILES)
      throw std::invalid_argument("SlabBatchNorm2DOp: one set of parameters per input");
    for (size_t r = 0; r < inputs.size(); ++r) {
      if (inputs[r]->shape() != inputs[0]->shape() || inputs[r]->batch_shape() != inputs[0]->batch_shape())
        throw std::invalid_argument("SlabBatchNorm2DOp: all tiles must have one shape");
      if (!inputs[r]->offset().is_zero())
        throw std::invalid_argument("SlabBatchNorm2DOp: input must be packed");
      xs_.push_back(inputs[r]->data());
      if (out_halo) {
        const typename V::Shape sh = inputs[r]->shape();
        ys_.push_back(VarData<V>(sh, typename V::Shape(out_halo, out_halo, 0),
                                 typename V::Shape(sh.shape[0] + 2 * out_halo, sh.shape[1] + 2 * out_halo, sh.shape[2]).packed_stride(),
                                 inputs[r]->batch_shape()));
      } else {
        ys_.push_back(VarData<V>(inputs[r]->shape(), inputs[r]->batch_shape()));
      }
      batch_mean_.push_back(vars[r].batch_mean->data());
      batch_variance_.push_back(vars[r].batch_variance->data());
      fixed_mean_.push_back(vars[r].fixed_mean->data());
      fixed_variance_.push_back(vars[r].fixed_variance->data());
      scale_.push_back(vars[r].scale->data());
      shift_.push_back(vars[r].shift->data());
      tmp_mean_.push_back(TxnVar<B>(_get_stat_shape(inputs[r]->shape())));
      tmp_variance_.push_back(TxnVar<B>(_get_stat_shape(inputs[r]->shape())));
    }
  }
  typename B::Shape _get_stat_shape(typename V::Shape in_shape) { return typename B::Shape(in_shape.shape[2]); }
  virtual void _push(EpochId e, function<void(Op *)> apply) {
    if (1 == stack_.push(e)) {
      for (size_t r = 0; r < x_vars_.size(); ++r) {
        x_vars_[r]->_push(e, apply);
        vars_[r].batch_mean->_push(e, apply);
        vars_[r].batch_variance->_push(e, apply);
        vars_[r].fixed_mean->_push(e, apply);
        vars_[r].fixed_variance->_push(e, apply);
        vars_[r].scale->_push(e, apply);
        vars_[r].shift->_push(e, apply);
      }
      apply(this);
    }
  }
  virtual void _pop(EpochId e, function<void(Op *)> apply) {
    if (stack_.degree(e) == stack_.pop(e)) {
      apply(this);
      for (size_t r = x_vars_.size(); r-- > 0;) {
        vars_[r].shift->_pop(e, apply);
        vars_[r].scale->_pop(e, apply);
        vars_[r].fixed_variance->_pop(e, apply);
        vars_[r].fixed_mean->_pop(e, apply);
        vars_[r].batch_variance->_pop(e, apply);
        vars_[r].batch_mean->_pop(e, apply);
        x_vars_[r]->_pop(e, apply);
      }
    }
  }
  virtual void _forward(TxnId txn);
  virtual void _backward(TxnId txn);
  virtual typename V::Shape shape() { return ys_[0].shape(); }
  virtual typename V::Shape offset() { return ys_[0].offset(); }
  virtual typename V::Shape stride() { return ys_[0].stride(); }
  virtual size_t batch_shape() { return ys_[0].batch_shape(); }
  virtual VarData<V> data() { return ys_[0].clone(); }

private:
  static void fill_sets(const RankVars &v, VarIdSet *params, VarIdSet *grads, VarIdSet *batch_stats, VarIdSet *fixed_stats) {
    batch_stats->insert(v.batch_mean->vars().at(0));
    batch_stats->insert(v.batch_variance->vars().at(0));
    fixed_stats->insert(v.fixed_mean->vars().at(0));
    fixed_stats->insert(v.fixed_variance->vars().at(0));
    params->insert(v.scale->vars().at(0));
    params->insert(v.shift->vars().at(0));
    grads->insert(v.scale->vars().at(1));
    grads->insert(v.shift->vars().at(1));
  }
  shared_ptr<Context> ctx_;
  shared_ptr<Switch> switch_var_;
  vector<shared_ptr<Var<V>>> x_vars_;
  vector<RankVars> vars_;
  vector<VarData<V>> xs_, ys_;
  vector<VarData<B>> batch_mean_, batch_variance_, fixed_mean_, fixed_variance_, scale_, shift_;
  vector<TxnVar<B>> tmp_mean_, tmp_variance_;
  bool relu_;
  size_t out_halo_;
};
template <typename Switch, typename V, typename B>
using CudnnBatchNorm2DOp = SlabBatchNorm2DOp<Switch, V, B>;

enum Activation {
  kReluAct,
};

// y = max(x, 0); backward dx += (y > 0 ? dy : 0) (src/op.cc:3189-3324, the out-of-place form)
template <typename V>
class CudnnActivationOp : public UnaryVarOp<V> {
public:
  static shared_ptr<Var<V>> Make(Activation activation, shared_ptr<Var<V>> input, shared_ptr<Context> ctx) {
    return make_shared<CudnnActivationOp<V>>(activation, input, ctx);
  }
  static vector<shared_ptr<Var<V>>> MakeParallel(Activation activation, vector<shared_ptr<Var<V>>> inputs,
                                                 shared_ptr<Context> ctx) {
    return make_per_rank<V>(ctx, [&](size_t r, shared_ptr<Context> dc) { return Make(activation, inputs.at(r), dc); });
  }
  CudnnActivationOp(Activation activation, shared_ptr<Var<V>> input, shared_ptr<Context> ctx) : UnaryVarOp<V>(input, ctx) {
    if (activation != kReluAct) throw std::invalid_argument("CudnnActivationOp: only kReluAct");
    if (!input->offset().is_zero()) throw std::invalid_argument("CudnnActivationOp: input must be packed");
    this->y_ = VarData<V>(input->shape(), input->batch_shape());
  }
  virtual void _forward(TxnId txn);
  virtual void _backward(TxnId txn);
};
template <typename V>
shared_ptr<Var<V>> relu(shared_ptr<Var<V>> input, shared_ptr<Context> ctx) {
  return CudnnActivationOp<V>::Make(kReluAct, input, ctx);
}
template <typename V>
vector<shared_ptr<Var<V>>> parallel_relu(vector<shared_ptr<Var<V>>> inputs, shared_ptr<Context> ctx) {
  return CudnnActivationOp<V>::MakeParallel(kReluAct, inputs, ctx);
}

// y = scale * x; backward dx += scale * dy (ScaleOp, src/op.cc:1221-1290)
template <typename T, typename V>
class ScaleOp : public UnaryVarOp<V> {
public:
  static shared_ptr<Var<V>> Make(T scale, shared_ptr<Var<V>> input, shared_ptr<Context> ctx) {
    return make_shared<ScaleOp<T, V>>(scale, input, ctx);
  }
  ScaleOp(T scale, shared_ptr<Var<V>> input, shared_ptr<Context> ctx) : UnaryVarOp<V>(input, ctx), scale_(scale) {
    if (!input->offset().is_zero()) throw std::invalid_argument("ScaleOp: input must be packed");
    this->y_ = VarData<V>(input->shape(), input->batch_shape());
  }
  virtual void _forward(TxnId txn);
  virtual void _backward(TxnId txn);

private:
  T scale_;
};

// y = x_0 + x_1 + ...; backward adds dy onto every input's gradient (JoinOp<V, SumJoin>, src/op.cc:744-867)
class SumJoin {};
template <typename V, typename Join>
class JoinOp : public virtual Op, public virtual Var<V> {
public:
  // sole_consumer_of (not in the reference): the index of an input that NO other node consumes, or -1.  The gradient
  // of such an input is the output's gradient and nothing else, so the output's gradient variable takes the
  // input's buffer and the backward pass copies nothing for it.  (An input that another node also consumes must not
  // be named: that node's contribution would land in the output's gradient and reach the other inputs.)
  // trunk_input (not in the reference): the index of an input that other nodes consume too, all of which lie
  // UPSTREAM of the join's remaining inputs (the block input of a residual block: its other consumer is the first
  // node of the path that ends in the join's second input), or -1.  Its gradient is the output's gradient plus what
  // those nodes add - and they run their backward pass after every node that reads the output's gradient, and add
  // in place.  So this input's gradient too can be the output's buffer: the gradient of a whole chain of residual
  // blocks is then one buffer that each block's first node adds to, and the sum's backward pass copies nothing.
  static shared_ptr<Var<V>> Make(Join join, vector<shared_ptr<Var<V>>> inputs, shared_ptr<Context> ctx,
                                 int sole_consumer_of = -1, int trunk_input = -1) {
    return make_shared<JoinOp<V, Join>>(join, false, inputs, ctx, sole_consumer_of, trunk_input);
  }
  // inputs.at(j).at(rank)
  static vector<shared_ptr<Var<V>>> MakeParallel(Join join, vector<vector<shared_ptr<Var<V>>>> inputs,
                                                 shared_ptr<Context> ctx, int sole_consumer_of = -1, int trunk_input = -1) {
    return make_per_rank<V>(ctx, [&](size_t r, shared_ptr<Context> dc) {
      vector<shared_ptr<Var<V>>> dev_inputs;
      for (auto &in : inputs) dev_inputs.push_back(in.at(r));
      return Make(join, dev_inputs, dc, sole_consumer_of, trunk_input);
    });
  }
  JoinOp(Join, bool in_place, vector<shared_ptr<Var<V>>> inputs, shared_ptr<Context> ctx, int sole_consumer_of = -1,
         int trunk_input = -1)
      : ctx_(ctx), inputs_(inputs) {
    if (in_place) throw std::invalid_argument("JoinOp: the in-place form is not part of this path");
    if (inputs.empty() || inputs.size() > ADH_MAX_TILES) throw std::invalid_argument("JoinOp: 1..16 inputs");
    for (auto &in : inputs) {
      if (in->shape() != inputs[0]->shape() || in->batch_shape() != inputs[0]->batch_shape() || !in->offset().is_zero())
        throw std::invalid_argument("JoinOp: inputs must be packed and of one shape");
      xs_.push_back(in->data());
    }
    y_ = VarData<V>(inputs[0]->shape(), inputs[0]->batch_shape());
    grad_shared_.assign(inputs.size(), false);
    if (sole_consumer_of >= 0) {
      if ((size_t)sole_consumer_of >= inputs.size()) throw std::invalid_argument("JoinOp: no such input");
      y_.alias_grad(xs_[(size_t)sole_consumer_of]);
      grad_shared_[(size_t)sole_consumer_of] = true;
    }
    if (trunk_input >= 0) {
      if ((size_t)trunk_input >= inputs.size() || trunk_input == sole_consumer_of) throw std::invalid_argument("JoinOp: no such input");
      // the nodes that hold copies of this input must see the shared buffer too: its variable forwards to the output's
      y_.absorb_grad(xs_[(size_t)trunk_input]);
      grad_shared_[(size_t)trunk_input] = true;
    }
  }
  virtual void _push(EpochId e, function<void(Op *)> apply) {
    if (1 == stack_.push(e)) {
      for (auto &in : inputs_) in->_push(e, apply);
      apply(this);
    }
  }
  virtual void _pop(EpochId e, function<void(Op *)> apply) {
    if (stack_.degree(e) == stack_.pop(e)) {
      apply(this);
      for (size_t j = inputs_.size(); j-- > 0;) inputs_[j]->_pop(e, apply);
    }
  }
  virtual void _forward(TxnId txn);
  virtual void _backward(TxnId txn);
  ARRAYDIFF_VAR_ACCESSORS(V)

private:
  shared_ptr<Context> ctx_;
  vector<shared_ptr<Var<V>>> inputs_;
  vector<VarData<V>> xs_;
  VarData<V> y_;
  vector<bool> grad_shared_;  // the input's gradient buffer is the output's
};
template <typename V>
shared_ptr<Var<V>> sum(vector<shared_ptr<Var<V>>> inputs, shared_ptr<Context> ctx) {
  return JoinOp<V, SumJoin>::Make(SumJoin(), inputs, ctx);
}
template <typename V>
vector<shared_ptr<Var<V>>> parallel_sum(vector<vector<shared_ptr<Var<V>>>> inputs, shared_ptr<Context> ctx,
                                        int sole_consumer_of = -1, int trunk_input = -1) {
  return JoinOp<V, SumJoin>::MakeParallel(SumJoin(), inputs, ctx, sole_consumer_of, trunk_input);
}

// ---------------------------------------------------------------------------
// pooling over the halo-padded slab
// ---------------------------------------------------------------------------
enum Pooling {
  kAveragePool,
  kMaxPool,
};

class Pool2DShape {
public:
  Pooling pooling;
  array<size_t, 2> axes;
  array<size_t, 2> window;
  array<size_t, 2> stride;
  array<size_t, 2> pad;
  bool halo_padded_input;
  // Not in the reference.  The inputs are the row tiles of one activation in rank order (a 1 x K grid) and carry
  // NO halo (halo_padded_input = false; pad is the zero padding of the unsplit pooling): the op is the reference's
  // HaloPad2DOp -> HaloExch2DOp -> pool chain in one node, and its input gradient comes out unpadded and complete.
  // The row split must stitch: tile height a multiple of the row stride, 0 < window - 2 * pad <= stride along the
  // rows, windows that reach the adjacent tiles only.
  bool unpadded_tiles = false;
};

// V = GPUBatchArray3D<float>.  With halo_padded_input the padded tile is pooled as a plain packed
// tensor with pad 0 (the halo holds the padding: neighbour rows after a halo exchange, zeros at the
// image border); without it the input must be packed and pad must be 0 (the global pooling before
// the classifier).  Implicit zero padding of an unpadded input is not part of this path and throws
// at construction.  One node serves all ranks it was made for: the K tiles go to the device in ONE
// launch per pass.
template <typename V>
class SlabPool2DOp : public virtual Op, public virtual Var<V> {
public:
  static shared_ptr<Var<V>> Make(Pool2DShape shape, shared_ptr<Var<V>> input, shared_ptr<Context> ctx) {
    return make_shared<SlabPool2DOp<V>>(shape, vector<shared_ptr<Var<V>>>{input}, ctx);
  }
  static vector<shared_ptr<Var<V>>> MakeParallel(Pool2DShape shape, vector<shared_ptr<Var<V>>> inputs,
                                                 shared_ptr<Context> ctx) {
    auto op = make_shared<SlabPool2DOp<V>>(shape, inputs, ctx);
    vector<shared_ptr<Var<V>>> outputs;
    for (size_t r = 0; r < inputs.size(); ++r) outputs.push_back(make_shared<NoOp<V>>(op, op->ys_.at(r).clone()));
    return outputs;
  }
  SlabPool2DOp(Pool2DShape shape, vector<shared_ptr<Var<V>>> inputs, shared_ptr<Context> ctx)
      : ctx_(ctx), shape_(shape), x_vars_(inputs) {
    if (shape.pooling != kAveragePool && shape.pooling != kMaxPool)
      throw std::invalid_argument("SlabPool2DOp: unknown pooling");
    if (shape.window[0] == 0 || shape.window[1] == 0 || shape.stride[0] == 0 || shape.stride[1] == 0)
      throw std::invalid_argument("SlabPool2DOp: empty window or stride");
    if (inputs.empty() || inputs.size() > ADH_MAX_TILES) throw std::invalid_argument("SlabPool2DOp: bad tile count");
    if (shape.unpadded_tiles) {
      const size_t tile_h = inputs[0]->shape().shape[1];
      if (shape.halo_padded_input || 2 * shape.pad[1] >= shape.window[1] || shape.window[1] - 2 * shape.pad[1] > shape.stride[1] ||
          tile_h % shape.stride[1] != 0 || shape.window[1] - 1 - shape.pad[1] > tile_h ||
          shape.pad[1] + (shape.window[1] - 1 - shape.pad[1]) / shape.stride[1] * shape.stride[1] > tile_h)
        throw std::invalid_argument("SlabPool2DOp: tiles without halo need a row split whose outputs stitch");
    } else if (!shape.halo_padded_input && (shape.pad[0] != 0 || shape.pad[1] != 0))
      throw std::invalid_argument("SlabPool2DOp: padding needs a halo-padded input");
    for (size_t r = 0; r < inputs.size(); ++r) {
      auto off = inputs[r]->offset();
      const size_t halo0 = shape.unpadded_tiles ? 0 : shape.pad[0], halo1 = shape.unpadded_tiles ? 0 : shape.pad[1];
      if (off.shape[0] != halo0 || off.shape[1] != halo1 || off.shape[2] != 0)
        throw std::invalid_argument("SlabPool2DOp: input halo must equal the pooling pad");
      if (inputs[r]->shape() != inputs[0]->shape() || inputs[r]->batch_shape() != inputs[0]->batch_shape())
        throw std::invalid_argument("SlabPool2DOp: all tiles must have one shape");
      xs_.push_back(inputs[r]->data());
      ys_.push_back(VarData<V>(_get_output_shape(inputs[r]->shape()), inputs[r]->batch_shape()));
    }
  }
  // out = floor((in + 2 pad - window) / stride) + 1 per axis, channels kept (what
  // cudnnGetPooling2dForwardOutputDim returns, op.cc:3346-3385)
  Shape3D _get_output_shape(Shape3D in_shape) {
    size_t out[2];
    for (int a = 0; a < 2; ++a) {
      const size_t padded = in_shape.shape[a] + 2 * shape_.pad[a];
      if (padded < shape_.window[a]) throw std::invalid_argument("SlabPool2DOp: window larger than the padded input");
      out[a] = (padded - shape_.window[a]) / shape_.stride[a] + 1;
    }
    return Shape3D(out[0], out[1], in_shape.shape[2]);
  }
  virtual void _push(EpochId e, function<void(Op *)> apply) {
    if (1 == stack_.push(e)) {
      for (auto &x : x_vars_) x->_push(e, apply);
      apply(this);
    }
  }
  virtual void _pop(EpochId e, function<void(Op *)> apply) {
    if (stack_.degree(e) == stack_.pop(e)) {
      apply(this);
      for (size_t r = x_vars_.size(); r-- > 0;) x_vars_[r]->_pop(e, apply);
    }
  }
  virtual void _forward(TxnId txn);
  virtual void _backward(TxnId txn);
  virtual typename V::Shape shape() { return ys_[0].shape(); }
  virtual typename V::Shape offset() { return ys_[0].offset(); }
  virtual typename V::Shape stride() { return ys_[0].stride(); }
  virtual size_t batch_shape() { return ys_[0].batch_shape(); }
  virtual VarData<V> data() { return ys_[0].clone(); }

private:
  shared_ptr<Context> ctx_;
  Pool2DShape shape_;
  vector<shared_ptr<Var<V>>> x_vars_;
  vector<VarData<V>> xs_;
  vector<VarData<V>> ys_;
};
template <typename V>
using CudnnPool2DOp = SlabPool2DOp<V>;

// ---------------------------------------------------------------------------
// softmax + negative log likelihood (1-D logits)
// ---------------------------------------------------------------------------
// (W, H, C) per example -> one vector of W*H*C per example, same order (parallel_flatten_nchw,
// src/zoo.cc:1861): a copy forward, an accumulation backward.
template <typename V, typename W>
class FlattenNCHWOp : public virtual Op, public virtual Var<W> {
public:
  static shared_ptr<Var<W>> Make(shared_ptr<Var<V>> input, shared_ptr<Context> ctx) {
    return make_shared<FlattenNCHWOp<V, W>>(input, ctx);
  }
  FlattenNCHWOp(shared_ptr<Var<V>> input, shared_ptr<Context> ctx)
      : ctx_(ctx), input_(input), x_(input->data()),
        y_(typename W::Shape(input->shape().flat_size()), input->batch_shape()) {
    if (!input->offset().is_zero()) throw std::invalid_argument("FlattenNCHWOp: input must be packed");
  }
  virtual void _push(EpochId e, function<void(Op *)> apply) {
    if (1 == stack_.push(e)) {
      input_->_push(e, apply);
      apply(this);
    }
  }
  virtual void _pop(EpochId e, function<void(Op *)> apply) {
    if (stack_.degree(e) == stack_.pop(e)) {
      apply(this);
      input_->_pop(e, apply);
    }
  }
  virtual void _forward(TxnId txn);
  virtual void _backward(TxnId txn);
  virtual typename W::Shape shape() { return y_.shape(); }
  virtual typename W::Shape offset() { return y_.offset(); }
  virtual typename W::Shape stride() { return y_.stride(); }
  virtual size_t batch_shape() { return y_.batch_shape(); }
  virtual VarData<W> data() { return y_.clone(); }

private:
  shared_ptr<Context> ctx_;
  shared_ptr<Var<V>> input_;
  VarData<V> x_;
  VarData<W> y_;
};

template <typename V, typename Label, typename Loss>
class SoftmaxNLLLossOp : public virtual Op, public virtual Var<Loss> {
public:
  SoftmaxNLLLossOp(shared_ptr<Var<V>> input, shared_ptr<Var<Label>> label, shared_ptr<Context> ctx)
      : ctx_(ctx), input_(input), label_var_(label), x_(input->data()), y_(input->shape(), input->batch_shape()),
        label_(label->data()), loss_(typename Loss::Shape(), input->batch_shape()) {}
  virtual void _push(EpochId e, function<void(Op *)> apply) {
    if (1 == stack_.push(e)) {
      input_->_push(e, apply);
      label_var_->_push(e, apply);
      apply(this);
    }
  }
  virtual void _pop(EpochId e, function<void(Op *)> apply) {
    if (stack_.degree(e) == stack_.pop(e)) {
      apply(this);
      label_var_->_pop(e, apply);
      input_->_pop(e, apply);
    }
  }
  virtual void _forward(TxnId txn);
  virtual void _backward(TxnId txn);
  // per-example losses: the sink gradient is 1 for every example (the reference reaches the
  // same through batch_sum + ScaleOp, src/zoo.cc:1877-1878)
  virtual void _set_grad_sink(TxnId txn) {
    GPUContext *c = gpu_ctx_of(ctx_);
    const float seed = sink_grad_;
    loss_.grad().accumulate(txn, id(), c, [c, seed](Loss *g) {
      GPUConn conn = c->conn();
      g->as_view().set_constant(seed, conn);
    });
  }
  // the gradient every example's loss is seeded with: 1 for the summed loss, 1/minibatch_size for
  // the mean the trainers minimise (the ScaleOp before batch_sum, src/zoo.cc:1877)
  void set_sink_grad(float g) { sink_grad_ = g; }
  template <typename T>
  void store_loss(TxnId txn, T *host) {
    GPUConn conn = gpu_ctx_of(ctx_)->conn();
    loss_.val().get(txn, id()).store_sync(host, conn);
  }
  template <typename T>
  void store_prob(TxnId txn, T *host) {
    GPUConn conn = gpu_ctx_of(ctx_)->conn();
    y_.val().get(txn, id()).store_sync(host, conn);
  }
  virtual typename Loss::Shape shape() { return loss_.shape(); }
  virtual typename Loss::Shape offset() { return loss_.offset(); }
  virtual typename Loss::Shape stride() { return loss_.stride(); }
  virtual size_t batch_shape() { return loss_.batch_shape(); }
  virtual VarData<Loss> data() { return loss_.clone(); }

private:
  shared_ptr<Context> ctx_;
  shared_ptr<Var<V>> input_;
  shared_ptr<Var<Label>> label_var_;
  VarData<V> x_;
  VarData<V> y_;  // softmax output, kept for backward
  VarData<Label> label_;
  VarData<Loss> loss_;
  float sink_grad_ = 1.0f;
};
template <typename V, typename Label, typename Loss>
using CudnnSoftmaxNLLLossOp = SoftmaxNLLLossOp<V, Label, Loss>;

template <typename V, typename Label, typename Loss>
shared_ptr<SoftmaxNLLLossOp<V, Label, Loss>> softmax_nll_loss(shared_ptr<Var<V>> input, shared_ptr<Var<Label>> label,
                                                              shared_ptr<Context> ctx) {
  return make_shared<SoftmaxNLLLossOp<V, Label, Loss>>(input, label, ctx);
}

// the float instantiations live in src/op.cc
typedef GPUBatchArray3D<float> Tile3f;
typedef GPUArray4D<float> Filter4f;

}  // namespace arraydiff

#endif
