// Learning-rate schedules, the Trainer loop and SGD (see deep8/Trainer.h for the reference lines).
#include "deep8/Trainer.h"

#include "deep8/Math.h"

namespace Deep8 {

float LearningRateIterator::next(int64_t) { DEEP8_RUNTIME_ERROR("can not call this function in LearningRateIterator"); }

ConstantLearningRateIterator::ConstantLearningRateIterator(float lr) : learningRate(lr) {}
float ConstantLearningRateIterator::next(int64_t) { return learningRate; }

LinearDecayLearningRateIterator::LinearDecayLearningRateIterator(int64_t total, float start, float end)
    : totalSteps(total), startLearningRate(start), endLearningRate(end) {}

float LinearDecayLearningRateIterator::next(int64_t steps) {
    return (float(steps) / float(totalSteps)) * (endLearningRate - startLearningRate) + startLearningRate;
}

Trainer::Trainer(LearningRateIterator *lr, float decay) : steps(0), learningRate(lr), weightDecay(decay) {}

void Trainer::update(Executor *, Variable *, float, float, int64_t) { DEEP8_RUNTIME_ERROR("can not call this function in trainer"); }

void Trainer::train(Executor *executor, std::vector<Variable *> parameters) {
    if (parameters.empty()) return;
    const float lr = learningRate->next(steps);
    for (auto parameter : parameters) {
        if (!parameter->updateGradient) continue;
        update(executor, parameter, lr, weightDecay, steps);
    }
    steps++;
}

void Trainer::train(Executor *executor) { train(executor, executor->trainableParameters()); }

SGDTrainer::SGDTrainer(LearningRateIterator *lr, float decay) : Trainer(lr, decay) {}

void SGDTrainer::update(Executor *, Variable *parameter, float learningRate, float weightDecay, int64_t) {
    Tensor value = parameter->value, gradient = parameter->gradient;
    const float alpha = -1 * learningRate;
    const float beta = 1.0f - learningRate * weightDecay;
    Math::AXPBY(gradient, alpha, value, beta, value);
}

AdamTrainer::AdamTrainer(LearningRateIterator *lr, float b1, float b2, float e, float decay)
    : Trainer(lr, decay), beta1(b1), beta2(b2), epsilon(e) {}

void AdamTrainer::update(Executor *executor, Variable *parameter, float learningRate, float weightDecay, int64_t steps) {
    Tensor value = parameter->value, gradient = parameter->gradient;
    if (m.find(parameter) == m.end()) {
        Variable *mt = executor->addVariable(value.shape, value.elementType, false);
        mt->value.zero();
        m[parameter] = mt;
    }
    if (v.find(parameter) == v.end()) {
        Variable *vt = executor->addVariable(value.shape, value.elementType, false);
        vt->value.zero();
        v[parameter] = vt;
    }
    Tensor mt = m[parameter]->value, vt = v[parameter]->value;
    Math::AdamUpdate(value, gradient, mt, vt, beta1, beta2, epsilon, learningRate, weightDecay, steps);
}

}  // namespace Deep8
