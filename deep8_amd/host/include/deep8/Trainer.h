// Trainers: walk the executor's trainable parameters and update each value from its gradient.
//   LearningRateIterator / Constant / LinearDecay   deep8/include/trainer/LearningRateIterator.h,
//       ConstantLearningRateIterator.h, LinearDecayLearningRateIterator.h (+ the .cpp of each)
//   Trainer       deep8/include/trainer/Trainer.h, deep8/src/trainer/Trainer.cpp:5-39
//   SGDTrainer    deep8/include/trainer/SGDTrainer.h, deep8/src/trainer/SGDTrainer.cpp:6-17
//                 value = (1 - lr * decay) * value - lr * gradient, one Math::AXPBY per parameter
//   AdamTrainer   deep8/include/trainer/AdamTrainer.h, deep8/src/trainer/AdamTrainer.cpp:6-33
#ifndef DEEP8_HOST_TRAINER_H
#define DEEP8_HOST_TRAINER_H

#include "deep8/Executor.h"

namespace Deep8 {

class LearningRateIterator {
public:
    virtual ~LearningRateIterator() = default;
    virtual float next(int64_t steps);
};

class ConstantLearningRateIterator : public LearningRateIterator {
public:
    float learningRate;
    explicit ConstantLearningRateIterator(float lr = 0.01);
    float next(int64_t steps) override;
};

class LinearDecayLearningRateIterator : public LearningRateIterator {
public:
    int64_t totalSteps;
    float startLearningRate;
    float endLearningRate;
    explicit LinearDecayLearningRateIterator(int64_t total, float start = 0.01, float end = 0);
    float next(int64_t steps) override;
};

class Trainer {
protected:
    int64_t steps;
    LearningRateIterator *learningRate;
    float weightDecay;  // l2 penalty
    explicit Trainer(LearningRateIterator *lr, float decay = 0);

public:
    virtual ~Trainer() = default;
    virtual void update(Executor *executor, Variable *parameter, float learningRate, float weightDecay, int64_t steps);
    void train(Executor *executor, std::vector<Variable *> parameters);
    void train(Executor *executor);
};

class SGDTrainer : public Trainer {
public:
    explicit SGDTrainer(LearningRateIterator *lr, float decay = 0);
    void update(Executor *executor, Variable *parameter, float learningRate, float weightDecay, int64_t steps) override;
};

// Adam with bias-corrected step size; the moment estimates are Variables the executor keeps
// (deep8/include/trainer/AdamTrainer.h, deep8/src/trainer/AdamTrainer.cpp:6-33).
class AdamTrainer : public Trainer {
public:
    float beta1;
    float beta2;
    float epsilon;
    std::unordered_map<Variable *, Variable *> m;
    std::unordered_map<Variable *, Variable *> v;

    explicit AdamTrainer(LearningRateIterator *lr, float beta1 = 0.9, float beta2 = 0.999, float epsilon = 1e-7, float decay = 0);
    void update(Executor *executor, Variable *parameter, float learningRate, float weightDecay, int64_t steps) override;
};

}  // namespace Deep8

#endif
