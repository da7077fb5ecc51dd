// The optimizer that drives a spatially-parallel graph: mirrors the reference's schedules, SGDConfig
// and ParallelSGDOptimizer (include/arraydiff/optimize.hh:19-136, 262-586) by name, constructor and
// method, on the one-GPU rank model of this library (ranks are row-tiles sharing one device and
// one in-order stream).
//
// What changes underneath:
//   - the per-rank gradient vectors are not reduced by a collective and then updated by three to
//     five axpy launches; ONE kernel reads all of them in rank order and writes momentum,
//     parameters and the lagged parameters (adh_sgd_step_f32);
//   - the root's updated vector is not broadcast: every rank's variables are loaded straight from
//     it (they live in the same memory);
//   - store_val / store_grad / load_val move all arrays of a rank with one launch each;
//   - the first compute batch of a step writes its gradients and statistics directly into the
//     accumulators instead of into a staging vector that is then copied.
// The values are those of the reference's sequence, with the rank sum taken in rank order.
#ifndef ARRAYDIFF_OPTIMIZE_HH
#define ARRAYDIFF_OPTIMIZE_HH

#include "arraydiff/context.hh"
#include "arraydiff/op.hh"

#include <algorithm>
#include <functional>
#include <memory>
#include <utility>

namespace arraydiff {

using std::function;
using std::pair;
using std::shared_ptr;

// A value per iteration number (optimize.hh:19-26).
template <typename T>
class Schedule {
public:
  virtual ~Schedule() {}
  virtual T at(size_t index) = 0;
};

template <typename T>
class ConstantSchedule : public virtual Schedule<T> {
public:
  explicit ConstantSchedule(T constant) : constant_(constant) {}
  virtual T at(size_t) { return constant_; }

private:
  T constant_;
};

// init until the first boundary, then the value attached to the last boundary at or below the
// index (optimize.hh:44-88)
template <typename T>
class PiecewiseStepSchedule : public virtual Schedule<T> {
public:
  explicit PiecewiseStepSchedule(T init) : init_(init) {}
  PiecewiseStepSchedule(T init, size_t step1, T val1) : init_(init), pieces_{{step1, val1}} {}
  PiecewiseStepSchedule(T init, size_t step1, T val1, size_t step2, T val2)
      : init_(init), pieces_{{step1, val1}, {step2, val2}} {}
  PiecewiseStepSchedule(T init, size_t step1, T val1, size_t step2, T val2, size_t step3, T val3)
      : init_(init), pieces_{{step1, val1}, {step2, val2}, {step3, val3}} {}
  PiecewiseStepSchedule(T init, vector<pair<size_t, T>> pieces) : init_(init), pieces_(pieces) {}
  virtual T at(size_t index) {
    T v = init_;
    for (const auto &piece : pieces_) {
      if (index < piece.first) break;
      v = piece.second;
    }
    return v;
  }

private:
  T init_;
  vector<pair<size_t, T>> pieces_;
};

// straight lines between (0, init) and the boundaries, constant after the last (optimize.hh:90-125)
template <typename T>
class PiecewiseLinearSchedule : public virtual Schedule<T> {
public:
  explicit PiecewiseLinearSchedule(T init) : init_(init) {}
  PiecewiseLinearSchedule(T init, size_t step1, T val1) : init_(init), pieces_{{step1, val1}} {}
  PiecewiseLinearSchedule(T init, vector<pair<size_t, T>> pieces) : init_(init), pieces_(pieces) {}
  virtual T at(size_t index) {
    size_t x0 = 0;
    T y0 = init_;
    for (const auto &piece : pieces_) {
      if (index < piece.first) {
        const T t = static_cast<T>(index - x0) / static_cast<T>(piece.first - x0);
        return y0 + t * (piece.second - y0);
      }
      x0 = piece.first;
      y0 = piece.second;
    }
    return y0;
  }

private:
  T init_;
  vector<pair<size_t, T>> pieces_;
};

// optimize.hh:127-136
class SGDConfig {
public:
  size_t minibatch_size;
  size_t compute_batch_size;
  shared_ptr<Schedule<double>> step_size;
  shared_ptr<Schedule<double>> momentum;
  bool nesterov;
  double l2_reg;
  double batch_norm_rate;
};

// params / grads / batch_stats / fixed_stats hold one VarIdSet per rank; every rank must span the
// same number of floats.  A variable shared by all ranks belongs in one rank's sets only (it is
// visited once per set it is a member of).
template <typename T>
class ParallelSGDOptimizer {
public:
  ParallelSGDOptimizer(SGDConfig cfg, shared_ptr<Op> sum_loss, vector<VarIdSet> params, vector<VarIdSet> grads,
                       vector<VarIdSet> batch_stats, vector<VarIdSet> fixed_stats)
      : num_ranks_(0), cfg_(cfg), iter_count_(0), sum_loss_(sum_loss), params_(params), grads_(grads),
        batch_stats_(batch_stats), fixed_stats_(fixed_stats), param_dim_(0), stat_dim_(0) {
    static_assert(sizeof(T) == 4, "the flat vectors are fp32");
    if (params.empty() || params.size() > ADH_MAX_TILES || params.size() != grads.size() ||
        params.size() != batch_stats.size() || params.size() != fixed_stats.size())
      throw std::invalid_argument("ParallelSGDOptimizer: one set of each kind per rank");
    if (cfg.minibatch_size == 0 || cfg.compute_batch_size == 0)
      throw std::invalid_argument("ParallelSGDOptimizer: empty batch");
  }

  size_t param_dim() const { return param_dim_; }
  size_t stat_dim() const { return stat_dim_; }
  size_t iter_count() const { return iter_count_; }
  // the root's flat vectors, for checkpoints and tests
  GPUMemory<T> &param() { return param_; }
  GPUMemory<T> &lagged_param() { return lagged_param_; }
  GPUMemory<T> &momentum_grad() { return momentum_grad_; }

  // optimize.hh:271-278: the current parameters into every rank's variables
  void reload_param(shared_ptr<Context> parallel_ctx) {
    (void)parallel_ctx;
    TxnId update_txn;
    for (size_t rank = 0; rank < num_ranks_; ++rank) expect(sum_loss_->load_val(update_txn, params_.at(rank), 0, &param_), param_dim_);
  }
  // optimize.hh:280-311: the parameters as they were before the look-ahead of a Nesterov step
  void reload_lagged_param(shared_ptr<Context> parallel_ctx) {
    (void)parallel_ctx;
    TxnId update_txn;
    for (size_t rank = 0; rank < num_ranks_; ++rank)
      expect(sum_loss_->load_val(update_txn, params_.at(rank), 0, &lagged_param_), param_dim_);
  }

  // optimize.hh:313-386.  The graph's parameters must hold their initial values (written in any
  // earlier transaction); rank 0's become every rank's.
  void reset(shared_ptr<Context> parallel_ctx) {
    MultiGPUContext *mgpu_ctx = mgpu_ctx_of(parallel_ctx);
    num_ranks_ = params_.size();
    if (num_ranks_ > mgpu_ctx->num_ranks()) throw std::invalid_argument("ParallelSGDOptimizer: more rank sets than ranks");
    {
      TxnId measure_txn;
      param_dim_ = sum_loss_->store_val(measure_txn, params_.at(0), 0, nullptr);
      stat_dim_ = sum_loss_->store_val(measure_txn, fixed_stats_.at(0), 0, nullptr);
      for (size_t rank = 0; rank < num_ranks_; ++rank) {
        expect(sum_loss_->store_val(measure_txn, params_.at(rank), 0, nullptr), param_dim_);
        expect(sum_loss_->store_grad(measure_txn, grads_.at(rank), 0, nullptr), param_dim_);
        expect(sum_loss_->store_val(measure_txn, fixed_stats_.at(rank), 0, nullptr), stat_dim_);
        expect(sum_loss_->store_val(measure_txn, batch_stats_.at(rank), 0, nullptr), stat_dim_);
      }
    }
    iter_count_ = 0;
    GPUContext *root = mgpu_ctx->device_context(0).get();
    param_ = GPUMemory<T>::Zeros(param_dim_, root);
    lagged_param_ = GPUMemory<T>::Zeros(param_dim_, root);
    momentum_grad_ = GPUMemory<T>::Zeros(param_dim_, root);
    batch_sum_grad_ = GPUMemory<T>();
    batch_stat_ = GPUMemory<T>();
    sum_grad_.clear();
    stat_.clear();
    avg_stat_.clear();
    running_stat_.clear();
    for (size_t rank = 0; rank < num_ranks_; ++rank) {
      GPUContext *dev = mgpu_ctx->device_context(rank).get();
      sum_grad_.push_back(GPUMemory<T>::Zeros(param_dim_, dev));
      stat_.push_back(GPUMemory<T>::Zeros(stat_dim_, dev));
      avg_stat_.push_back(GPUMemory<T>::Zeros(stat_dim_, dev));
      running_stat_.push_back(GPUMemory<T>::Zeros(stat_dim_, dev));
    }
    TxnId init_txn;
    for (size_t rank = 0; rank < num_ranks_; ++rank) {
      sum_loss_->persist(init_txn, params_.at(rank));
      sum_loss_->persist(init_txn, fixed_stats_.at(rank));
    }
    expect(sum_loss_->store_val(init_txn, params_.at(0), 0, &param_), param_dim_);
    GPUConn conn = root->conn();
    lagged_param_.copy(param_, param_dim_, 0, 0, conn);
    for (size_t rank = 1; rank < num_ranks_; ++rank) expect(sum_loss_->load_val(init_txn, params_.at(rank), 0, &param_), param_dim_);
  }

  // optimize.hh:388-559.  compute_batch_fn(txn, batch_size, sum_loss) feeds one compute batch and
  // runs forward and backward in transaction txn (persisting the parameters into it first).
  void step(function<void(TxnId, size_t, shared_ptr<Op>)> &compute_batch_fn, shared_ptr<Context> parallel_ctx) {
    MultiGPUContext *mgpu_ctx = mgpu_ctx_of(parallel_ctx);
    if (num_ranks_ == 0) throw std::logic_error("ParallelSGDOptimizer: step before reset");
    GPUContext *root = mgpu_ctx->device_context(0).get();
    GPUConn conn = root->conn();
    const size_t num_batches = (cfg_.minibatch_size + cfg_.compute_batch_size - 1) / cfg_.compute_batch_size;
    for (size_t batch_nr = 0; batch_nr < num_batches; ++batch_nr) {
      TxnId batch_txn;
      const size_t actual_batch_size = std::min(cfg_.compute_batch_size, cfg_.minibatch_size - batch_nr * cfg_.compute_batch_size);
      compute_batch_fn(batch_txn, actual_batch_size, sum_loss_);
      if (0 == batch_nr) {
        // the parameters the gradients were taken at (optimize.hh:394-400; all ranks hold the same)
        expect(sum_loss_->store_val(batch_txn, params_.at(0), 0, &param_), param_dim_);
        for (size_t rank = 0; rank < num_ranks_; ++rank) {
          expect(sum_loss_->store_grad(batch_txn, grads_.at(rank), 0, &sum_grad_.at(rank)), param_dim_);
          expect(sum_loss_->store_val(batch_txn, batch_stats_.at(rank), 0, &avg_stat_.at(rank)), stat_dim_);
        }
      } else {
        if (batch_sum_grad_.size() < param_dim_) batch_sum_grad_ = GPUMemory<T>::Zeros(param_dim_, root);
        if (batch_stat_.size() < stat_dim_) batch_stat_ = GPUMemory<T>::Zeros(stat_dim_, root);
        const T alpha = T(1) / static_cast<T>(batch_nr + 1);
        for (size_t rank = 0; rank < num_ranks_; ++rank) {
          expect(sum_loss_->store_grad(batch_txn, grads_.at(rank), 0, &batch_sum_grad_), param_dim_);
          sum_grad_.at(rank).add(batch_sum_grad_, param_dim_, 0, 0, conn);
          expect(sum_loss_->store_val(batch_txn, batch_stats_.at(rank), 0, &batch_stat_), stat_dim_);
          if (stat_dim_) avg_stat_.at(rank).add_online(alpha, batch_stat_, stat_dim_, 0, 0, conn);
        }
      }
    }

    // rank sum + l2 + momentum + update + lagged copy (optimize.hh:443-497)
    const float mu = static_cast<float>(cfg_.momentum->at(iter_count_));
    const float alpha = static_cast<float>(cfg_.step_size->at(iter_count_));
    const float next_alpha = cfg_.nesterov ? static_cast<float>(cfg_.step_size->at(iter_count_ + 1)) : alpha;
    const float *grads[ADH_MAX_TILES];
    for (size_t rank = 0; rank < num_ranks_; ++rank) grads[rank] = sum_grad_.at(rank).dptr();
    adh_check(adh_sgd_step_f32(param_dim_, (uint32_t)num_ranks_, grads, static_cast<float>(cfg_.l2_reg), mu, alpha,
                               next_alpha, cfg_.nesterov ? 1 : 0, param_.dptr(), momentum_grad_.dptr(),
                               lagged_param_.dptr(), sum_grad_.at(0).dptr(), conn.stream()),
              "ParallelSGDOptimizer::step");
    // running statistics of every rank (optimize.hh:507-514)
    const float epsilon = static_cast<float>(cfg_.batch_norm_rate);
    for (size_t rank = 0; rank < num_ranks_; ++rank)
      adh_check(adh_stat_step_f32(stat_dim_, epsilon, avg_stat_.at(rank).dptr(), running_stat_.at(rank).dptr(),
                                  stat_.at(rank).dptr(), conn.stream()),
                "ParallelSGDOptimizer::step (statistics)");

    // the root's parameters into every rank (the reference's broadcast + load, optimize.hh:518-556)
    TxnId update_txn;
    for (size_t rank = 0; rank < num_ranks_; ++rank) {
      expect(sum_loss_->load_val(update_txn, params_.at(rank), 0, &param_), param_dim_);
      if (stat_dim_) expect(sum_loss_->load_val(update_txn, fixed_stats_.at(rank), 0, &stat_.at(rank)), stat_dim_);
    }
    ++iter_count_;
  }

private:
  static void expect(size_t got, size_t want) {
    if (got != want) throw std::logic_error("ParallelSGDOptimizer: ranks span different numbers of floats");
  }
  size_t num_ranks_;
  SGDConfig cfg_;
  size_t iter_count_;
  shared_ptr<Op> sum_loss_;
  vector<VarIdSet> params_, grads_, batch_stats_, fixed_stats_;
  size_t param_dim_, stat_dim_;
  GPUMemory<T> param_, lagged_param_, momentum_grad_, batch_sum_grad_, batch_stat_;
  vector<GPUMemory<T>> sum_grad_, stat_, avg_stat_, running_stat_;
};

}  // namespace arraydiff

#endif
