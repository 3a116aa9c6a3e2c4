// Trainers: walk the executor's trainable parameters and update each value from its gradient.
//   LearningRateIterator / Constant / LinearDecay   deep8/include/trainer/LearningRateIterator.h,
//       ConstantLearningRateIterator.h, LinearDecayLearningRateIterator.h (+ the .cpp of each)
//   Trainer       deep8/include/trainer/Trainer.h, deep8/src/trainer/Trainer.cpp:5-39
//   SGDTrainer    deep8/include/trainer/SGDTrainer.h, deep8/src/trainer/SGDTrainer.cpp:6-17
//                 value = (1 - lr * decay) * value - lr * gradient, one Math::AXPBY per parameter
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

}  // namespace Deep8

#endif
