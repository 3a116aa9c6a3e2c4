// Executor / EagerExecutor: owns the device, creates Variables, runs each Function as it is
// added and drives the breadth-first backward pass.
//   Executor        deep8/include/model/Executor.h:27-137, deep8/src/model/Executor.cpp:9-324
//   EagerExecutor   deep8/src/model/EagerExecutor.cpp:8-93
//   Net sugar       deep8/include/model/Net.h:41-167 (parameter, inputParameter, feed, fetch,
//                   operator*, operator+, operator-, matrixMultiply, conv2d, deConv2d, l1Norm, l2Norm,
//                   reduceMean, l1NormLoss, l2NormLoss, backward)
// Only DeviceType::GPU can be constructed in this build.
#ifndef DEEP8_HOST_EXECUTOR_H
#define DEEP8_HOST_EXECUTOR_H

#include <unordered_map>
#include <unordered_set>

#include "deep8/Nodes.h"

namespace Deep8 {

enum class NameType {
    Node = 0, Variable, Function, Conv2d_Weight, Conv2d_Bias, DeConv2d_Weight, DeConv2d_Bias, MatrixMultiply_Weight,
};

class Executor {
protected:
    int64_t uniqueId;
    std::unordered_map<std::string, int64_t> nameUniqueId;
    std::unordered_set<std::string> uniqueNames;
    Device *device;
    std::unordered_map<std::string, Node *> allNodes;
    std::unordered_map<std::string, Variable *> retainVariables;  // parameters: survive backward()
    std::unordered_map<std::string, Node *> interimNodes;         // deleted after backward()

    explicit Executor(DeviceType deviceType = DeviceType::GPU);

    void initDeviceGPU();
    std::string namePrefix(NameType nameType);
    std::string generateUniqueName(NameType nameType);
    int64_t generateUniqueId();
    Tensor createTensor(Shape &shape, DType type);
    Tensor createTensor(Shape &shape, ElementType type);
    Tensor createTensorGPU(Shape &shape, ElementType type);
    Variable *createVariableByFunction(Function *func);

public:
    virtual ~Executor();

    Device *getDevice() { return device; }
    void removeGradient();

    Variable *addVariable(Shape &shape, ElementType type, bool updateGradient = true, bool retain = true);
    Variable *addVariable(std::vector<size_t> list, ElementType type, bool updateGradient = true, bool retain = true);
    Variable *addVariable(size_t batch, std::vector<size_t> list, ElementType type, bool updateGradient = true, bool retain = true);
    Variable *addVariable(Shape &shape, DType type, bool updateGradient = true, bool retain = true);
    Variable *addVariable(std::vector<size_t> list, DType type, bool updateGradient = true, bool retain = true);
    Variable *addVariable(size_t batch, std::vector<size_t> list, DType type, bool updateGradient = true, bool retain = true);
    Variable *addVariable(std::string name, Shape &shape, DType type, bool updateGradient = true, bool retain = true);
    Variable *addVariable(std::string name, size_t batch, std::vector<size_t> list, DType type, bool updateGradient = true, bool retain = true);

    void clearInterimNodes();
    Node *nodeByName(std::string name);
    Variable *retainVariableByName(std::string name);
    std::vector<Variable *> trainableParameters();

    virtual Variable *addFunction(Function *func);
    virtual void forward(Node *last);
    virtual void backward(Node *last, bool clearInterim = true);
};

class EagerExecutor : public Executor {
public:
    explicit EagerExecutor(DeviceType deviceType = DeviceType::GPU);
    Variable *addFunction(Function *func) override;
    void forward(Node *last) override;
    void backward(Node *last, bool clearInterim = true) override;
};

// ---- Net.h sugar for the path ---------------------------------------------------------------
void backward(Variable &v, bool clearInterim = true);
void backward(Variable *v, bool clearInterim = true);
Variable &parameter(Executor *executor, std::vector<size_t> list, bool updateGradient = true, DType type = DType::Float32);
Variable &parameter(Executor *executor, size_t batch, std::vector<size_t> list, bool updateGradient = true, DType type = DType::Float32);
Variable &inputParameter(Executor *executor, std::vector<size_t> list, DType type = DType::Float32);
Variable &inputParameter(Executor *executor, size_t batch, std::vector<size_t> list, DType type = DType::Float32);
Variable &feed(Variable &v, const void *ptr);
Variable &fetch(Variable &v, void *ptr);
Variable &operator*(Variable &x, Variable &y);  // MatrixMultiply
Variable &matrixMultiply(Variable &x, Variable &y);
Variable &conv2d(Variable &x, Variable &filter, bool covered = true, int strideY = 1, int strideX = 1, int dilationY = 1, int dilationX = 1);
Variable &deConv2d(Variable &x, Variable &filter, bool covered = false, int strideY = 1, int strideX = 1);
Variable &operator+(Variable &x, Variable &y);  // Add, with broadcasting
Variable &add(Variable &x, Variable &y);
Variable &relu(Variable &x);
Variable &matrixMultiplyBiasReLu(Variable &x, Variable &y, Variable &bias);  // relu(x * y + bias) as one node
Variable &conv2dBiasReLu(Variable &x, Variable &filter, Variable &bias, bool covered = true, int strideY = 1, int strideX = 1, int dilationY = 1, int dilationX = 1);
Variable &operator-(Variable &x, Variable &y);  // Minus, with broadcasting
Variable &minus(Variable &x, Variable &y);
Variable &l1Norm(Variable &x);
Variable &l2Norm(Variable &x);
Variable &reduceMean(Variable &x, std::vector<int> axis = {-1}, bool keepDims = true);
Variable &l1NormLoss(Variable &x);
Variable &l2NormLoss(Variable &x);

}  // namespace Deep8

#endif
