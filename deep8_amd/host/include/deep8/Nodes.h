// Graph nodes: Node, Variable, Function and the three Function subclasses on the dense-contraction
// path.  Same public surface as the reference:
//   Node / OutputEntry   deep8/include/nodes/Node.h:29-80, deep8/include/model/OutputEntry.h:10-30
//   Variable             deep8/include/nodes/Variable.h:9-53 (+ feed/fetch and the three op builders)
//   Function             deep8/include/nodes/Function.h:46-65, deep8/src/nodes/Function.cpp:41-102
//   MatrixMultiply       deep8/src/nodes/MatrixMultiply.cpp:6-52
//   Conv2d               deep8/src/nodes/Conv2d.cpp:6-152
//   DeConv2d             deep8/src/nodes/DeConv2d.cpp:6-126
#ifndef DEEP8_HOST_NODES_H
#define DEEP8_HOST_NODES_H

#include <unordered_map>

#include "deep8/Model.h"

namespace Deep8 {

class Executor;
class Node;

enum class NodeType { Unknow = 0, Variable, Function };

class OutputEntry {
public:
    std::unordered_map<Node *, size_t> entries;  // consumer -> which of its inputs this node is
    void add(Node *node, size_t i);
    void remove(Node *node);
    void clear();
    size_t size();
    Node *first();
};

class Node {
public:
    NodeType type;
    int64_t id;
    std::string name;
    Executor *executor;  // may be nullptr (nodes built by hand, as the tests do)
    std::vector<Node *> inputs;
    OutputEntry outputs;

protected:
    Node();
    explicit Node(Node *input);
    explicit Node(std::vector<Node *> &inputs);
    Node(int64_t id, std::string name, Executor *exe);
    Node(int64_t id, std::string name, Executor *exe, Node *input);
    Node(int64_t id, std::string name, Executor *exe, std::vector<Node *> &inputs);

public:
    virtual ~Node();
    virtual void forward();
    virtual void backward();
    virtual std::string toString();
};

class Variable : public Node {
public:
    Tensor value;
    Tensor gradient;
    bool updateGradient;

protected:
    Variable(int64_t id, std::string name, Executor *exe);

public:
    Variable(int64_t id, std::string name, Executor *exe, Tensor &v);
    Variable(int64_t id, std::string name, Executor *exe, Tensor &v, Tensor &g);
    Variable(int64_t id, std::string name, Executor *exe, Node *input);
    Variable(int64_t id, std::string name, Executor *exe, Node *input, Tensor &v);
    Variable(int64_t id, std::string name, Executor *exe, Node *input, Tensor &v, Tensor &g);

    Shape shape();
    ElementType elementType();
    DeviceType deviceType();
    bool isScalar();
    void zeroGradient();
    void oneGradient();
    void removeGradient();
    void forward() override;   // nothing to do
    void backward() override;  // nothing to do
    std::string valueStr();

    Variable &feed(const void *hostPtr);  // host -> value
    Variable &fetch(void *hostPtr);       // value -> host (blocking)
    Variable &constant(float scalar = 0);
    Variable &zero();
    Variable &one();

    // graph builders of the dense-contraction path (need an executor)
    Variable &matrixMultiply(Variable &y);
    Variable &conv2d(Variable &filter, bool covered = true, int strideY = 1, int strideX = 1, int dilationY = 1, int dilationX = 1);
    Variable &deConv2d(Variable &filter, bool covered = false, int strideY = 1, int strideX = 1);
    // the element-wise steps that follow them
    Variable &add(Variable &y);
    Variable &relu();
    // ... and the three as one node: relu(this * y + bias), relu(conv2d(this, filter) + bias); bias has one value per
    // element of the result's last dimension
    Variable &matrixMultiplyBiasReLu(Variable &y, Variable &bias);
    Variable &conv2dBiasReLu(Variable &filter, Variable &bias, bool covered = true, int strideY = 1, int strideX = 1, int dilationY = 1, int dilationX = 1);
    // what a loss needs (deep8/src/nodes/Variable.cpp:342-346,461-465,521-535)
    Variable &minus(Variable &y);
    Variable &l1Norm();
    Variable &l2Norm();
    Variable &reduceMean(std::vector<int> axis = {-1}, bool keepDims = true);
    Variable &l1NormLoss();  // l1Norm().reduceMean({}, false)
    Variable &l2NormLoss();  // l2Norm().reduceMean({}, false)
    // value ~ N(mean, stddev) drawn on the host and copied over (deep8/src/nodes/Variable.cpp:201-205; the
    // reference draws on the device from an unseeded generator, so only the distribution is comparable)
    Variable &gaussian(float mean = 0.0, float stddev = 0.01);
    // pooling (deep8/src/nodes/Variable.cpp: maxPooling2d / avgPooling2d)
    Variable &maxPooling2d(bool covered = false, int filterHeight = 1, int filterWidth = 1, int strideY = 1, int strideX = 1);
    Variable &avgPooling2d(bool covered = false, int filterHeight = 1, int filterWidth = 1, int strideY = 1, int strideX = 1);
};

enum class FunctionType { Unkown = 0, Conv2d, DeConv2d, MatrixMultiply, Add, ReLu, Minus, L1Norm, L2Norm, ReduceMean, MaxPooling2d, AvgPooling2d,
                          MatrixMultiplyBiasReLu, Conv2dBiasReLu };

class Function : public Node {
protected:
    explicit Function(std::vector<Node *> &inputs);

public:
    virtual bool isShared();
    virtual Shape checkShape(std::vector<Shape> &inputShapes);
    virtual ElementType checkElementType(std::vector<ElementType> &inputTypes);

    virtual void forward(const std::vector<const Tensor *> &inputs, Tensor *output);
    virtual void backward(const std::vector<const Tensor *> &inputs, const Tensor *output,
                          const Tensor *outputGradient, size_t index, Tensor *iGradient);

    void forward() override;   // gathers the input Variables' values, writes the output Variable
    void backward() override;  // one backward(..., i, ...) per input that wants a gradient
};

class MatrixMultiply : public Function {
public:
    explicit MatrixMultiply(std::vector<Node *> &inputs, size_t inputCount = 2);
    Shape checkShape(std::vector<Shape> &inputShapes) override;
    ElementType checkElementType(std::vector<ElementType> &inputTypes) override;
    void forward(const std::vector<const Tensor *> &inputs, Tensor *output) override;
    void backward(const std::vector<const Tensor *> &inputs, const Tensor *output, const Tensor *outputGradient,
                  size_t index, Tensor *iGradient) override;
    void backward() override;  // both gradients through one Math call when both inputs take one
};

class Conv2d : public Function {
public:
    bool covered;
    int strideY, strideX, dilationY, dilationX;

    explicit Conv2d(std::vector<Node *> &inputs, bool covered = true, int strideY = 1, int strideX = 1,
                    int dilationY = 1, int dilationX = 1, size_t inputCount = 2);
    Shape checkShape(std::vector<Shape> &inputShapes) override;
    ElementType checkElementType(std::vector<ElementType> &inputTypes) override;
    void forward(const std::vector<const Tensor *> &inputs, Tensor *output) override;
    void backward(const std::vector<const Tensor *> &inputs, const Tensor *output, const Tensor *outputGradient,
                  size_t index, Tensor *iGradient) override;
    void backward() override;  // both gradients through one Math call when both inputs take one
};

class DeConv2d : public Function {
public:
    bool forwardCovered;
    int forwardStrideY, forwardStrideX;

    explicit DeConv2d(std::vector<Node *> &inputs, bool covered = false, int strideY = 1, int strideX = 1);
    Shape checkShape(std::vector<Shape> &inputShapes) override;
    ElementType checkElementType(std::vector<ElementType> &inputTypes) override;
    void forward(const std::vector<const Tensor *> &inputs, Tensor *output) override;
    void backward(const std::vector<const Tensor *> &inputs, const Tensor *output, const Tensor *outputGradient,
                  size_t index, Tensor *iGradient) override;
    void backward() override;  // both gradients through one Math call when both inputs take one
};

// z = x + y under numpy's broadcasting rule (deep8/include/nodes/Add.h:8-27, deep8/src/nodes/Add.cpp:6-45)
class Add : public Function {
public:
    explicit Add(std::vector<Node *> &inputs);
    Shape checkShape(std::vector<Shape> &inputShapes) override;
    ElementType checkElementType(std::vector<ElementType> &inputTypes) override;
    void forward(const std::vector<const Tensor *> &inputs, Tensor *output) override;
    void backward(const std::vector<const Tensor *> &inputs, const Tensor *output, const Tensor *outputGradient,
                  size_t index, Tensor *iGradient) override;
};

// y = max(x, 0) (deep8/include/nodes/ReLu.h:8-26, deep8/src/nodes/ReLu.cpp:6-33)
class ReLu : public Function {
public:
    explicit ReLu(std::vector<Node *> &inputs);
    Shape checkShape(std::vector<Shape> &inputShapes) override;
    ElementType checkElementType(std::vector<ElementType> &inputTypes) override;
    void forward(const std::vector<const Tensor *> &inputs, Tensor *output) override;
    void backward(const std::vector<const Tensor *> &inputs, const Tensor *output, const Tensor *outputGradient,
                  size_t index, Tensor *iGradient) override;
};

// relu(x * y + bias) and relu(conv2d(x, filter) + bias) as ONE node each (inputs: x, y / filter, bias): the forward
// pass is one call whose product kernel adds the bias and cuts at zero in its own store; the backward pass gates
// the output gradient and sums the bias gradient in one pass, then runs the contraction's two gradient products on
// the gated gradient.  Same values as the chain MatrixMultiply / Conv2d -> Add -> ReLu of separate nodes
// (deep8/src/nodes/MatrixMultiply.cpp, Conv2d.cpp, Add.cpp, ReLu.cpp); no counterpart in the reference, whose
// eager executor runs every node as it is created.
class MatrixMultiplyBiasReLu : public MatrixMultiply {
public:
    explicit MatrixMultiplyBiasReLu(std::vector<Node *> &inputs);
    Shape checkShape(std::vector<Shape> &inputShapes) override;
    ElementType checkElementType(std::vector<ElementType> &inputTypes) override;
    void forward(const std::vector<const Tensor *> &inputs, Tensor *output) override;
    // one input at a time (gates the output gradient anew on every call)
    void backward(const std::vector<const Tensor *> &inputs, const Tensor *output, const Tensor *outputGradient,
                  size_t index, Tensor *iGradient) override;
    using Function::forward;
    void backward() override;  // all inputs that want a gradient, gating once
};

class Conv2dBiasReLu : public Conv2d {
public:
    explicit Conv2dBiasReLu(std::vector<Node *> &inputs, bool covered = true, int strideY = 1, int strideX = 1,
                            int dilationY = 1, int dilationX = 1);
    Shape checkShape(std::vector<Shape> &inputShapes) override;
    ElementType checkElementType(std::vector<ElementType> &inputTypes) override;
    void forward(const std::vector<const Tensor *> &inputs, Tensor *output) override;
    void backward(const std::vector<const Tensor *> &inputs, const Tensor *output, const Tensor *outputGradient,
                  size_t index, Tensor *iGradient) override;
    using Function::forward;
    void backward() override;
};

// z = x - y under the same broadcasting rule (deep8/include/nodes/Minus.h, deep8/src/nodes/Minus.cpp:6-39)
class Minus : public Function {
public:
    explicit Minus(std::vector<Node *> &inputs);
    Shape checkShape(std::vector<Shape> &inputShapes) override;
    ElementType checkElementType(std::vector<ElementType> &inputTypes) override;
    void forward(const std::vector<const Tensor *> &inputs, Tensor *output) override;
    void backward(const std::vector<const Tensor *> &inputs, const Tensor *output, const Tensor *outputGradient,
                  size_t index, Tensor *iGradient) override;
};

// y[b] = sum |x[b]| and y[b] = sqrt(sum x[b]^2), output Shape(batch, {1})
// (deep8/src/nodes/L1Norm.cpp:6-38, deep8/src/nodes/L2Norm.cpp:6-36)
class L1Norm : public Function {
public:
    explicit L1Norm(std::vector<Node *> &inputs);
    Shape checkShape(std::vector<Shape> &inputShapes) override;
    ElementType checkElementType(std::vector<ElementType> &inputTypes) override;
    void forward(const std::vector<const Tensor *> &inputs, Tensor *output) override;
    void backward(const std::vector<const Tensor *> &inputs, const Tensor *output, const Tensor *outputGradient,
                  size_t index, Tensor *iGradient) override;
};

class L2Norm : public Function {
public:
    explicit L2Norm(std::vector<Node *> &inputs);
    Shape checkShape(std::vector<Shape> &inputShapes) override;
    ElementType checkElementType(std::vector<ElementType> &inputTypes) override;
    void forward(const std::vector<const Tensor *> &inputs, Tensor *output) override;
    void backward(const std::vector<const Tensor *> &inputs, const Tensor *output, const Tensor *outputGradient,
                  size_t index, Tensor *iGradient) override;
};

// mean over `axis` (0 is the batch axis, empty = all) (deep8/src/nodes/ReduceMean.cpp:7-75)
class ReduceMean : public Function {
public:
    std::vector<int> axis;
    bool keepDims;

    explicit ReduceMean(std::vector<Node *> &inputs, std::vector<int> reduceAxis = {-1}, bool keep = true);
    Shape checkShape(std::vector<Shape> &inputShapes) override;
    ElementType checkElementType(std::vector<ElementType> &inputTypes) override;
    void forward(const std::vector<const Tensor *> &inputs, Tensor *output) override;
    void backward(const std::vector<const Tensor *> &inputs, const Tensor *output, const Tensor *outputGradient,
                  size_t index, Tensor *iGradient) override;
};

// Pooling over [B, H, W, C] (deep8/src/nodes/MaxPooling2d.cpp, deep8/src/nodes/AvgPooling2d.cpp)
class Pooling2d : public Function {
public:
    bool isMax;
    bool covered;
    int filterHeight, filterWidth, strideY, strideX;

    Pooling2d(std::vector<Node *> &inputs, bool isMax, bool covered, int filterHeight, int filterWidth, int strideY, int strideX);
    Shape checkShape(std::vector<Shape> &inputShapes) override;
    ElementType checkElementType(std::vector<ElementType> &inputTypes) override;
    void forward(const std::vector<const Tensor *> &inputs, Tensor *output) override;
    void backward(const std::vector<const Tensor *> &inputs, const Tensor *output, const Tensor *outputGradient,
                  size_t index, Tensor *iGradient) override;
};

class MaxPooling2d : public Pooling2d {
public:
    explicit MaxPooling2d(std::vector<Node *> &inputs, bool covered = false, int filterHeight = 1, int filterWidth = 1, int strideY = 1, int strideX = 1)
        : Pooling2d(inputs, true, covered, filterHeight, filterWidth, strideY, strideX) {}
};

class AvgPooling2d : public Pooling2d {
public:
    explicit AvgPooling2d(std::vector<Node *> &inputs, bool covered = false, int filterHeight = 1, int filterWidth = 1, int strideY = 1, int strideX = 1)
        : Pooling2d(inputs, false, covered, filterHeight, filterWidth, strideY, strideX) {}
};

// Shape of x + y (deep8/include/utils/ShapeUtils.h:19-36)
Shape broadcastShape(const Shape &shape1, const Shape &shape2);

}  // namespace Deep8

#endif
