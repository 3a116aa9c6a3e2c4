// Node, Variable, Function and the MatrixMultiply / Conv2d / DeConv2d functions (see deep8/Nodes.h).
#include "deep8/Nodes.h"

#include <algorithm>
#include <random>

#include "deep8/Executor.h"
#include "deep8/Math.h"

namespace Deep8 {

// ---- OutputEntry ---------------------------------------------------------------------------------------
void OutputEntry::add(Node *node, size_t i) {
    DEEP8_ARGUMENT_CHECK(nullptr != node, "the node can not be nullptr");
    entries[node] = i;
}
void OutputEntry::remove(Node *node) { entries.erase(node); }
void OutputEntry::clear() { entries.clear(); }
size_t OutputEntry::size() { return entries.size(); }
Node *OutputEntry::first() {
    DEEP8_ARGUMENT_CHECK(!entries.empty(), "the outputs is empty");
    return entries.begin()->first;
}

// ---- Node ---------------------------------------------------------------------------------------------------
Node::Node() : type(NodeType::Unknow), id(-1), executor(nullptr) {}

Node::Node(Node *input) : Node() {
    inputs.push_back(input);
    input->outputs.add(this, 0);
}

Node::Node(std::vector<Node *> &in) : Node() {
    inputs = in;
    for (size_t i = 0; i < inputs.size(); ++i) inputs[i]->outputs.add(this, i);
}

Node::Node(int64_t i, std::string n, Executor *exe) : type(NodeType::Unknow), id(i), name(std::move(n)), executor(exe) {}

Node::Node(int64_t i, std::string n, Executor *exe, Node *input) : Node(i, std::move(n), exe) {
    inputs.push_back(input);
    input->outputs.add(this, 0);
}

Node::Node(int64_t i, std::string n, Executor *exe, std::vector<Node *> &in) : Node(i, std::move(n), exe) {
    inputs = in;
    for (size_t k = 0; k < inputs.size(); ++k) inputs[k]->outputs.add(this, k);
}

Node::~Node() {}
void Node::forward() { DEEP8_RUNTIME_ERROR("Can not call this function from Node"); }
void Node::backward() { DEEP8_RUNTIME_ERROR("Can not call this function from Node"); }
std::string Node::toString() { return "Node: the Base class of Function and Variable"; }

// ---- Variable --------------------------------------------------------------------------------------------------
static void checkPair(const Tensor &value, const Tensor &gradient) {
    DEEP8_ARGUMENT_CHECK(value.deviceType() == gradient.deviceType(), "the values and gradient must be the same type");
    DEEP8_ARGUMENT_CHECK(value.elementType == gradient.elementType, "the values and gradient data type must be the same");
    DEEP8_ARGUMENT_CHECK(value.shape == gradient.shape, "the shape of Value and Gradient must be same");
}

Variable::Variable(int64_t id, std::string name, Executor *exe) : Node(id, std::move(name), exe), updateGradient(false) {
    type = NodeType::Variable;
}

Variable::Variable(int64_t id, std::string name, Executor *exe, Tensor &v)
    : Node(id, std::move(name), exe), value(v), updateGradient(false) {
    type = NodeType::Variable;
}

Variable::Variable(int64_t id, std::string name, Executor *exe, Tensor &v, Tensor &g)
    : Node(id, std::move(name), exe), value(v), gradient(g), updateGradient(true) {
    checkPair(value, gradient);
    type = NodeType::Variable;
}

Variable::Variable(int64_t id, std::string name, Executor *exe, Node *input)
    : Node(id, std::move(name), exe, input), updateGradient(false) {
    type = NodeType::Variable;
}

Variable::Variable(int64_t id, std::string name, Executor *exe, Node *input, Tensor &v)
    : Node(id, std::move(name), exe, input), value(v), updateGradient(false) {
    type = NodeType::Variable;
}

Variable::Variable(int64_t id, std::string name, Executor *exe, Node *input, Tensor &v, Tensor &g)
    : Node(id, std::move(name), exe, input), value(v), gradient(g), updateGradient(true) {
    checkPair(value, gradient);
    type = NodeType::Variable;
}

Shape Variable::shape() {
    if (updateGradient) DEEP8_ARGUMENT_CHECK(value.shape == gradient.shape, "the value and gradient shape must be same");
    return value.shape;
}

ElementType Variable::elementType() {
    if (updateGradient)
        DEEP8_ARGUMENT_CHECK(value.elementType == gradient.elementType, "the value and gradient elementType must be same");
    return value.elementType;
}

DeviceType Variable::deviceType() {
    if (updateGradient)
        DEEP8_ARGUMENT_CHECK(value.deviceType() == gradient.deviceType(), "the value and gradient deviceType must be same");
    return value.deviceType();
}

bool Variable::isScalar() { return updateGradient ? value.isScalar() && gradient.isScalar() : value.isScalar(); }

void Variable::zeroGradient() {
    DEEP8_ARGUMENT_CHECK(updateGradient, "this variable does not have gradient");
    // a gradient that owns its whole allocation is zeroed lazily: the first routine that would add
    // into it overwrites instead, any other access fills it first (Device::zeroLater)
    if (0 == gradient.offset && gradient.byteCount() == gradient.storage.size)
        gradient.device()->zeroLater(gradient.storage.ptr, gradient.storage.size);
    else
        Math::Constant(gradient, 0);
}

void Variable::oneGradient() {
    DEEP8_ARGUMENT_CHECK(updateGradient, "this variable does not have gradient");
    Math::Constant(gradient, 1);
}

void Variable::removeGradient() {
    if (updateGradient) {
        gradient = Tensor();
        updateGradient = false;
    }
}

void Variable::forward() {}
void Variable::backward() {}
std::string Variable::valueStr() { return value.valueStr(); }

Variable &Variable::feed(const void *ptr) {
    DEEP8_ARGUMENT_CHECK(nullptr != ptr, "the pointer can not be null");
    value.device()->copyFromCPUToGPU(ptr, value.raw(), value.byteCount());
    return *this;
}

Variable &Variable::fetch(void *ptr) {
    DEEP8_ARGUMENT_CHECK(nullptr != ptr, "the pointer can not be null");
    value.device()->copyFromGPUToCPU(value.raw(), ptr, value.byteCount());
    return *this;
}

Variable &Variable::constant(float scalar) {
    Math::Constant(value, scalar);
    return *this;
}
Variable &Variable::zero() { return constant(0); }
Variable &Variable::one() { return constant(1); }

Variable &Variable::matrixMultiply(Variable &y) {
    DEEP8_ARGUMENT_CHECK(nullptr != executor, "the Variable does not belong to an Executor");
    std::vector<Node *> in = {this, &y};
    return *executor->addFunction(new MatrixMultiply(in));
}

Variable &Variable::add(Variable &y) {
    DEEP8_ARGUMENT_CHECK(nullptr != executor, "the Variable does not belong to an Executor");
    std::vector<Node *> in = {this, &y};
    return *executor->addFunction(new Add(in));
}

Variable &Variable::relu() {
    DEEP8_ARGUMENT_CHECK(nullptr != executor, "the Variable does not belong to an Executor");
    std::vector<Node *> in = {this};
    return *executor->addFunction(new ReLu(in));
}

Variable &Variable::matrixMultiplyBiasReLu(Variable &y, Variable &bias) {
    DEEP8_ARGUMENT_CHECK(nullptr != executor, "the Variable does not belong to an Executor");
    std::vector<Node *> in = {this, &y, &bias};
    return *executor->addFunction(new MatrixMultiplyBiasReLu(in));
}

Variable &Variable::conv2dBiasReLu(Variable &filter, Variable &bias, bool covered, int strideY, int strideX, int dilationY, int dilationX) {
    DEEP8_ARGUMENT_CHECK(nullptr != executor, "the Variable does not belong to an Executor");
    std::vector<Node *> in = {this, &filter, &bias};
    return *executor->addFunction(new Conv2dBiasReLu(in, covered, strideY, strideX, dilationY, dilationX));
}

Variable &Variable::minus(Variable &y) {
    DEEP8_ARGUMENT_CHECK(nullptr != executor, "the Variable does not belong to an Executor");
    std::vector<Node *> in = {this, &y};
    return *executor->addFunction(new Minus(in));
}

Variable &Variable::l1Norm() {
    DEEP8_ARGUMENT_CHECK(nullptr != executor, "the Variable does not belong to an Executor");
    std::vector<Node *> in = {this};
    return *executor->addFunction(new L1Norm(in));
}

Variable &Variable::l2Norm() {
    DEEP8_ARGUMENT_CHECK(nullptr != executor, "the Variable does not belong to an Executor");
    std::vector<Node *> in = {this};
    return *executor->addFunction(new L2Norm(in));
}

Variable &Variable::reduceMean(std::vector<int> axis, bool keepDims) {
    DEEP8_ARGUMENT_CHECK(nullptr != executor, "the Variable does not belong to an Executor");
    std::vector<Node *> in = {this};
    return *executor->addFunction(new ReduceMean(in, axis, keepDims));
}

Variable &Variable::l1NormLoss() { return l1Norm().reduceMean({}, false); }
Variable &Variable::l2NormLoss() { return l2Norm().reduceMean({}, false); }

Variable &Variable::gaussian(float mean, float stddev) {
    DEEP8_ARGUMENT_CHECK(DType::Float32 == value.elementType.id, "gaussian() fills Float32 variables");
    static std::mt19937 engine{std::random_device{}()};
    std::normal_distribution<float> dist(mean, stddev);
    std::vector<float> host(value.shape.size());
    for (auto &v : host) v = dist(engine);
    return feed(host.data());
}

Variable &Variable::maxPooling2d(bool covered, int filterHeight, int filterWidth, int strideY, int strideX) {
    DEEP8_ARGUMENT_CHECK(nullptr != executor, "the Variable does not belong to an Executor");
    std::vector<Node *> in = {this};
    return *executor->addFunction(new MaxPooling2d(in, covered, filterHeight, filterWidth, strideY, strideX));
}

Variable &Variable::avgPooling2d(bool covered, int filterHeight, int filterWidth, int strideY, int strideX) {
    DEEP8_ARGUMENT_CHECK(nullptr != executor, "the Variable does not belong to an Executor");
    std::vector<Node *> in = {this};
    return *executor->addFunction(new AvgPooling2d(in, covered, filterHeight, filterWidth, strideY, strideX));
}

Variable &Variable::conv2d(Variable &filter, bool covered, int strideY, int strideX, int dilationY, int dilationX) {
    DEEP8_ARGUMENT_CHECK(nullptr != executor, "the Variable does not belong to an Executor");
    std::vector<Node *> in = {this, &filter};
    return *executor->addFunction(new Conv2d(in, covered, strideY, strideX, dilationY, dilationX));
}

Variable &Variable::deConv2d(Variable &filter, bool covered, int strideY, int strideX) {
    DEEP8_ARGUMENT_CHECK(nullptr != executor, "the Variable does not belong to an Executor");
    std::vector<Node *> in = {this, &filter};
    return *executor->addFunction(new DeConv2d(in, covered, strideY, strideX));
}

// ---- Function -----------------------------------------------------------------------------------------------------
Function::Function(std::vector<Node *> &in) : Node(in) { type = NodeType::Function; }

bool Function::isShared() { return false; }
Shape Function::checkShape(std::vector<Shape> &) { return Shape(); }

ElementType Function::checkElementType(std::vector<ElementType> &inputTypes) {
    if (inputTypes.empty()) return ElementType::unknown();
    for (size_t i = 1; i < inputTypes.size(); ++i)
        DEEP8_ARGUMENT_CHECK(inputTypes[0] == inputTypes[i], "the input's ElementType must be same");
    return inputTypes[0];
}

void Function::forward(const std::vector<const Tensor *> &, Tensor *) {
    DEEP8_RUNTIME_ERROR("can not call this forward by Function class");
}

void Function::backward(const std::vector<const Tensor *> &, const Tensor *, const Tensor *, size_t, Tensor *) {
    DEEP8_RUNTIME_ERROR("can not call this backward by Function class");
}

// Collect the input Variables' value tensors, all on the output's device.
static std::vector<const Tensor *> gatherInputs(Function *f, Variable *&outputVar) {
    for (Node *n : f->inputs) DEEP8_ARGUMENT_CHECK(NodeType::Variable == n->type, "the inputs must be a Variable type");
    DEEP8_ARGUMENT_CHECK(1 == f->outputs.size(), "the output size must be 1");
    DEEP8_ARGUMENT_CHECK(NodeType::Variable == f->outputs.first()->type, "the output must be a Variable type");
    outputVar = (Variable *)f->outputs.first();
    const DeviceType dev = outputVar->deviceType();
    std::vector<const Tensor *> values;
    for (Node *n : f->inputs) {
        Variable *v = (Variable *)n;
        DEEP8_ARGUMENT_CHECK(dev == v->deviceType(), "the device of input must be same with output");
        values.push_back(&v->value);
    }
    return values;
}

void Function::forward() {
    Variable *out = nullptr;
    std::vector<const Tensor *> values = gatherInputs(this, out);
    this->forward(values, &out->value);
}

void Function::backward() {
    Variable *out = nullptr;
    std::vector<const Tensor *> values = gatherInputs(this, out);
    for (size_t i = 0; i < inputs.size(); ++i) {
        Variable *in = (Variable *)inputs[i];
        if (in->updateGradient) this->backward(values, &out->value, &out->gradient, i, &in->gradient);
    }
}

// ---- MatrixMultiply ---------------------------------------------------------------------------------------------------
MatrixMultiply::MatrixMultiply(std::vector<Node *> &in, size_t count) : Function(in) {
    DEEP8_ARGUMENT_CHECK(count == inputs.size(), "the MatrixMultiply Function needs 2 input (3 with a bias)");
}

Shape MatrixMultiply::checkShape(std::vector<Shape> &inputShapes) {
    DEEP8_ARGUMENT_CHECK(2 == inputShapes.size(), "the input count must be 2");
    const Shape &x = inputShapes[0], &y = inputShapes[1];
    DEEP8_ARGUMENT_CHECK(x.batch == y.batch || 1 == x.batch || 1 == y.batch, "the batch of input is error");
    DEEP8_ARGUMENT_CHECK((1 == x.nDims || 2 == x.nDims) && (1 == y.nDims || 2 == y.nDims), "the inputs dimensions is error");
    DEEP8_ARGUMENT_CHECK(x.col() == y.row(), "the col of input1 must same to the row of input2");
    const size_t batch = std::max(x.batch, y.batch);
    if (1 == y.col()) return Shape(batch, {x.row()});  // a 1-D result
    return Shape(batch, {x.row(), y.col()});
}

ElementType MatrixMultiply::checkElementType(std::vector<ElementType> &inputTypes) {
    DEEP8_ARGUMENT_CHECK(2 == inputTypes.size(), "the input count must be 2");
    return Function::checkElementType(inputTypes);
}

void MatrixMultiply::forward(const std::vector<const Tensor *> &in, Tensor *output) {
    Math::MatrixMultiply(*in[0], *in[1], *output);
}

void MatrixMultiply::backward(const std::vector<const Tensor *> &in, const Tensor *output, const Tensor *outputGradient,
                              size_t index, Tensor *iGradient) {
    if (0 == index) Math::MatrixMultiplyGradX(*in[0], *iGradient, *in[1], *output, *outputGradient);
    else if (1 == index) Math::MatrixMultiplyGradY(*in[0], *in[1], *iGradient, *output, *outputGradient);
    else DEEP8_RUNTIME_ERROR("the index is error");
}

// Both inputs take a gradient (the usual case): one Math call for the two products, which the library may run as one
// launch.  The two gradients must be different tensors (x * x has one input twice: its two products add into the same
// gradient, one after the other).
void MatrixMultiply::backward() {
    Variable *a = (Variable *)inputs[0], *b = (Variable *)inputs[1];
    if (2 != inputs.size() || !a->updateGradient || !b->updateGradient || a == b) return Function::backward();
    Variable *out = nullptr;
    std::vector<const Tensor *> values = gatherInputs(this, out);
    Math::MatrixMultiplyGradXY(*values[0], a->gradient, *values[1], b->gradient, out->value, out->gradient);
}

// ---- Conv2d / DeConv2d ---------------------------------------------------------------------------------------------------
// An interim buffer from the device pool for one Math call; freed as soon as the call has
// queued its kernels (single stream + a pool that never gives memory back while alive).
namespace {
struct Interim {
    Device *device;
    void *ptr;
    Interim(Device *d, size_t bytes) : device(d), ptr(d->malloc(bytes)) {}
    ~Interim() { device->free(ptr); }
};

void checkConvInputs(std::vector<Shape> &inputShapes) {
    DEEP8_ARGUMENT_CHECK(2 == inputShapes.size(), "the input count must be 2");
    const Shape &in = inputShapes[0], &filter = inputShapes[1];
    DEEP8_ARGUMENT_CHECK(3 == in.nDims, "Conv2d needs inputs nDims is 3");
    DEEP8_ARGUMENT_CHECK(4 == filter.nDims && 1 == filter.batch, "Conv2d needs filter nDims is 4, the batch must be 1");
    DEEP8_ARGUMENT_CHECK(in.dim(2) == filter.dim(3), "the inputs dimension is error");
    DEEP8_ARGUMENT_CHECK(filter.dim(1) > 0 && filter.dim(2) > 0, "the filter width and height must bigger than 0");
}
}  // namespace

Conv2d::Conv2d(std::vector<Node *> &in, bool cov, int sy, int sx, int dy, int dx, size_t count)
    : Function(in), covered(cov), strideY(sy), strideX(sx), dilationY(dy), dilationX(dx) {
    DEEP8_ARGUMENT_CHECK(count == inputs.size(), "the Conv2d Function needs 2 input (3 with a bias)");
    DEEP8_ARGUMENT_CHECK(strideY >= 1 && strideX >= 1, "the stride can not smaller than 1");
    DEEP8_ARGUMENT_CHECK(dilationY >= 1 && dilationX >= 1, "the dilation can not smaller than 1");
}

Shape Conv2d::checkShape(std::vector<Shape> &inputShapes) {
    checkConvInputs(inputShapes);
    const Shape &in = inputShapes[0], &filter = inputShapes[1];
    const int FH = (int)filter.dim(1), FW = (int)filter.dim(2), IH = (int)in.dim(0), IW = (int)in.dim(1);
    if (!covered)
        DEEP8_ARGUMENT_CHECK(FH <= IH && FW <= IW, "the not covered mode Padding type needs filter smaller than input");
    const int realFH = FH + (FH - 1) * (dilationY - 1), realFW = FW + (FW - 1) * (dilationX - 1);
    const int OH = covered ? (IH - 1) / strideY + 1 : (IH - realFH) / strideY + 1;
    const int OW = covered ? (IW - 1) / strideX + 1 : (IW - realFW) / strideX + 1;
    DEEP8_ARGUMENT_CHECK(OH > 0 && OW > 0, "the output height or width must > 0");
    return Shape(in.batch, {(size_t)OH, (size_t)OW, filter.dim(0)});
}

ElementType Conv2d::checkElementType(std::vector<ElementType> &inputTypes) {
    DEEP8_ARGUMENT_CHECK(2 == inputTypes.size(), "the input count must be 2");
    return Function::checkElementType(inputTypes);
}

void Conv2d::forward(const std::vector<const Tensor *> &in, Tensor *output) {
    Interim buf(output->device(),
                Math::Conv2dInterimSize(*in[0], *in[1], *output, covered, strideY, strideX, dilationY, dilationX));
    Math::Conv2d(*in[0], *in[1], *output, covered, strideY, strideX, dilationY, dilationX, buf.ptr);
}

void Conv2d::backward(const std::vector<const Tensor *> &in, const Tensor *output, const Tensor *outputGradient,
                      size_t index, Tensor *iGradient) {
    if (0 == index) {
        Interim buf(iGradient->device(), Math::Conv2dGradXInterimSize(*in[0], *iGradient, *in[1], *output, *outputGradient,
                                                                      covered, strideY, strideX, dilationY, dilationX));
        Math::Conv2dGradX(*in[0], *iGradient, *in[1], *output, *outputGradient, covered, strideY, strideX, dilationY,
                          dilationX, buf.ptr);
    } else if (1 == index) {
        Interim buf(iGradient->device(), Math::Conv2dGradYInterimSize(*in[0], *in[1], *iGradient, *output, *outputGradient,
                                                                      covered, strideY, strideX, dilationY, dilationX));
        Math::Conv2dGradY(*in[0], *in[1], *iGradient, *output, *outputGradient, covered, strideY, strideX, dilationY,
                          dilationX, buf.ptr);
    } else {
        DEEP8_RUNTIME_ERROR("the index is error");
    }
}

// Input and filter both take a gradient (the usual case inside a network): one Math call for the two products, which
// the library runs as one launch on a small layer.  (Conv2dBiasReLu has its own backward().)
void Conv2d::backward() {
    Variable *a = (Variable *)inputs[0], *b = (Variable *)inputs[1];
    if (2 != inputs.size() || !a->updateGradient || !b->updateGradient || a == b) return Function::backward();
    Variable *out = nullptr;
    std::vector<const Tensor *> values = gatherInputs(this, out);
    Math::Conv2dGradXY(*values[0], a->gradient, *values[1], b->gradient, out->value, out->gradient, covered, strideY, strideX,
                       dilationY, dilationX);
}

DeConv2d::DeConv2d(std::vector<Node *> &in, bool cov, int sy, int sx)
    : Function(in), forwardCovered(cov), forwardStrideY(sy), forwardStrideX(sx) {
    DEEP8_ARGUMENT_CHECK(2 == inputs.size(), "the DeConv2d Function needs 2 input");
    DEEP8_ARGUMENT_CHECK(forwardStrideY >= 1 && forwardStrideX >= 1, "the stride is error");
}

Shape DeConv2d::checkShape(std::vector<Shape> &inputShapes) {
    checkConvInputs(inputShapes);
    const Shape &in = inputShapes[0], &filter = inputShapes[1];
    const int FH = (int)filter.dim(1), FW = (int)filter.dim(2), IH = (int)in.dim(0), IW = (int)in.dim(1);
    // the inverse of Conv2d's size rule
    const int OH = (IH - 1) * forwardStrideY + (forwardCovered ? 1 : FH);
    const int OW = (IW - 1) * forwardStrideX + (forwardCovered ? 1 : FW);
    DEEP8_ARGUMENT_CHECK(OH > 0 && OW > 0, "the output height/width must > 0");
    return Shape(in.batch, {(size_t)OH, (size_t)OW, filter.dim(0)});
}

ElementType DeConv2d::checkElementType(std::vector<ElementType> &inputTypes) {
    DEEP8_ARGUMENT_CHECK(2 == inputTypes.size(), "the input count must be 2");
    return Function::checkElementType(inputTypes);
}

void DeConv2d::forward(const std::vector<const Tensor *> &in, Tensor *output) {
    Interim buf(output->device(),
                Math::DeConv2dInterimSize(*in[0], *in[1], *output, forwardCovered, forwardStrideY, forwardStrideX));
    Math::DeConv2d(*in[0], *in[1], *output, forwardCovered, forwardStrideY, forwardStrideX, buf.ptr);
}

void DeConv2d::backward(const std::vector<const Tensor *> &in, const Tensor *output, const Tensor *outputGradient,
                        size_t index, Tensor *iGradient) {
    if (0 == index) {
        Interim buf(iGradient->device(), Math::DeConv2dGradXInterimSize(*in[0], *iGradient, *in[1], *output, *outputGradient,
                                                                        forwardCovered, forwardStrideY, forwardStrideX));
        Math::DeConv2dGradX(*in[0], *iGradient, *in[1], *output, *outputGradient, forwardCovered, forwardStrideY,
                            forwardStrideX, buf.ptr);
    } else if (1 == index) {
        Interim buf(iGradient->device(), Math::DeConv2dGradYInterimSize(*in[0], *in[1], *iGradient, *output, *outputGradient,
                                                                        forwardCovered, forwardStrideY, forwardStrideX));
        Math::DeConv2dGradY(*in[0], *in[1], *iGradient, *output, *outputGradient, forwardCovered, forwardStrideY,
                            forwardStrideX, buf.ptr);
    } else {
        DEEP8_RUNTIME_ERROR("the index of DeConv2d backward is error");
    }
}

void DeConv2d::backward() {
    Variable *a = (Variable *)inputs[0], *b = (Variable *)inputs[1];
    if (2 != inputs.size() || !a->updateGradient || !b->updateGradient || a == b) return Function::backward();
    Variable *out = nullptr;
    std::vector<const Tensor *> values = gatherInputs(this, out);
    Math::DeConv2dGradXY(*values[0], a->gradient, *values[1], b->gradient, out->value, out->gradient, forwardCovered, forwardStrideY,
                         forwardStrideX);
}

// ---- contraction + bias + ReLu as one node ---------------------------------------------------------------------------
namespace {
// a tensor of t's shape and type from t's device pool (released with its last copy)
Tensor tensorLike(const Tensor &t) {
    Device *dev = t.device();
    const size_t bytes = t.byteCount();
    void *ptr = dev->malloc(bytes);
    size_t *ref = (size_t *)dev->mallocCPU(sizeof(size_t));
    TensorStorage storage(ptr, ref, bytes, dev);
    Shape shape = t.shape;
    return Tensor(storage, 0, shape, t.elementType);
}

void checkBiasShape(const Shape &bias, const Shape &out) {
    DEEP8_ARGUMENT_CHECK(1 == bias.batch && 1 == bias.nDims && bias.dim(0) == out.dim(out.nDims - 1),
                         "the bias needs one value per element of the output's last dimension");
}

// The backward pass shared by the two fused nodes: gate once, then the products the inputs ask for -- both from one
// Math call (`both`) when the two operands are different variables that each take a gradient, else one by one.
template <typename Products, typename Both>
void fusedBackward(Function *f, const std::vector<const Tensor *> &values, Variable *out, const Products &products, const Both &both) {
    Variable *bias = (Variable *)f->inputs[2];
    Tensor dpre = tensorLike(out->gradient);
    if (bias->updateGradient) {
        Math::BiasReLuGrad(out->value, out->gradient, dpre, bias->gradient);
    } else {
        Tensor unused = tensorLike(bias->value);
        Math::BiasReLuGrad(out->value, out->gradient, dpre, unused);
    }
    Variable *a = (Variable *)f->inputs[0], *b = (Variable *)f->inputs[1];
    if (a->updateGradient && b->updateGradient && a != b) {
        both(values, out->value, dpre, a->gradient, b->gradient);
        return;
    }
    for (size_t i = 0; i < 2; ++i) {
        Variable *in = (Variable *)f->inputs[i];
        if (in->updateGradient) products(values, &out->value, &dpre, i, &in->gradient);
    }
}
}  // namespace

MatrixMultiplyBiasReLu::MatrixMultiplyBiasReLu(std::vector<Node *> &in) : MatrixMultiply(in, 3) {}

Shape MatrixMultiplyBiasReLu::checkShape(std::vector<Shape> &inputShapes) {
    DEEP8_ARGUMENT_CHECK(3 == inputShapes.size(), "the input count must be 3");
    std::vector<Shape> two(inputShapes.begin(), inputShapes.begin() + 2);
    const Shape out = MatrixMultiply::checkShape(two);
    checkBiasShape(inputShapes[2], out);
    return out;
}

ElementType MatrixMultiplyBiasReLu::checkElementType(std::vector<ElementType> &inputTypes) {
    DEEP8_ARGUMENT_CHECK(3 == inputTypes.size(), "the input count must be 3");
    return Function::checkElementType(inputTypes);
}

void MatrixMultiplyBiasReLu::forward(const std::vector<const Tensor *> &in, Tensor *output) {
    Math::MatrixMultiplyBiasReLu(*in[0], *in[1], *in[2], *output);
}

void MatrixMultiplyBiasReLu::backward(const std::vector<const Tensor *> &in, const Tensor *output, const Tensor *outputGradient,
                                      size_t index, Tensor *iGradient) {
    DEEP8_ARGUMENT_CHECK(index < 3, "the index is error");
    Tensor dpre = tensorLike(*outputGradient);
    if (2 == index) {
        Math::BiasReLuGrad(*output, *outputGradient, dpre, *iGradient);
        return;
    }
    Tensor unused = tensorLike(*in[2]);
    Math::BiasReLuGrad(*output, *outputGradient, dpre, unused);
    MatrixMultiply::backward(in, output, &dpre, index, iGradient);
}

void MatrixMultiplyBiasReLu::backward() {
    Variable *out = nullptr;
    std::vector<const Tensor *> values = gatherInputs(this, out);
    fusedBackward(this, values, out, [this](const std::vector<const Tensor *> &v, const Tensor *z, const Tensor *dz, size_t i, Tensor *g) {
        MatrixMultiply::backward(v, z, dz, i, g);
    }, [](const std::vector<const Tensor *> &v, const Tensor &z, const Tensor &dz, Tensor &gx, Tensor &gy) {
        Math::MatrixMultiplyGradXY(*v[0], gx, *v[1], gy, z, dz);
    });
}

Conv2dBiasReLu::Conv2dBiasReLu(std::vector<Node *> &in, bool cov, int sy, int sx, int dy, int dx) : Conv2d(in, cov, sy, sx, dy, dx, 3) {}

Shape Conv2dBiasReLu::checkShape(std::vector<Shape> &inputShapes) {
    DEEP8_ARGUMENT_CHECK(3 == inputShapes.size(), "the input count must be 3");
    std::vector<Shape> two(inputShapes.begin(), inputShapes.begin() + 2);
    const Shape out = Conv2d::checkShape(two);
    checkBiasShape(inputShapes[2], out);
    return out;
}

ElementType Conv2dBiasReLu::checkElementType(std::vector<ElementType> &inputTypes) {
    DEEP8_ARGUMENT_CHECK(3 == inputTypes.size(), "the input count must be 3");
    return Function::checkElementType(inputTypes);
}

void Conv2dBiasReLu::forward(const std::vector<const Tensor *> &in, Tensor *output) {
    Interim buf(output->device(),
                Math::Conv2dInterimSize(*in[0], *in[1], *output, covered, strideY, strideX, dilationY, dilationX));
    Math::Conv2dBiasReLu(*in[0], *in[1], *in[2], *output, covered, strideY, strideX, dilationY, dilationX, buf.ptr);
}

void Conv2dBiasReLu::backward(const std::vector<const Tensor *> &in, const Tensor *output, const Tensor *outputGradient,
                              size_t index, Tensor *iGradient) {
    DEEP8_ARGUMENT_CHECK(index < 3, "the index is error");
    Tensor dpre = tensorLike(*outputGradient);
    if (2 == index) {
        Math::BiasReLuGrad(*output, *outputGradient, dpre, *iGradient);
        return;
    }
    Tensor unused = tensorLike(*in[2]);
    Math::BiasReLuGrad(*output, *outputGradient, dpre, unused);
    Conv2d::backward(in, output, &dpre, index, iGradient);
}

void Conv2dBiasReLu::backward() {
    Variable *out = nullptr;
    std::vector<const Tensor *> values = gatherInputs(this, out);
    fusedBackward(this, values, out, [this](const std::vector<const Tensor *> &v, const Tensor *z, const Tensor *dz, size_t i, Tensor *g) {
        Conv2d::backward(v, z, dz, i, g);
    }, [this](const std::vector<const Tensor *> &v, const Tensor &z, const Tensor &dz, Tensor &gx, Tensor &gw) {
        Math::Conv2dGradXY(*v[0], gx, *v[1], gw, z, dz, covered, strideY, strideX, dilationY, dilationX);
    });
}

// ---- Add / ReLu -------------------------------------------------------------------------------------------------
Shape broadcastShape(const Shape &shape1, const Shape &shape2) {
    DEEP8_ARGUMENT_CHECK(1 == shape1.batch || 1 == shape2.batch || shape1.batch == shape2.batch, "the batch must be 1 or equal");
    const size_t nDims = std::max<size_t>(shape1.nDims, shape2.nDims);
    std::vector<size_t> ret(nDims);
    for (int i = (int)nDims - 1, i1 = (int)shape1.nDims - 1, i2 = (int)shape2.nDims - 1; i >= 0; --i, --i1, --i2) {
        const size_t size1 = i1 >= 0 ? shape1.dim(i1) : 1, size2 = i2 >= 0 ? shape2.dim(i2) : 1;
        DEEP8_ARGUMENT_CHECK(1 == size1 || 1 == size2 || size1 == size2, "the Shape can not Broadcast");
        ret[i] = std::max<size_t>(size1, size2);
    }
    return Shape(std::max<size_t>(shape1.batch, shape2.batch), ret);
}

Add::Add(std::vector<Node *> &in) : Function(in) {
    DEEP8_ARGUMENT_CHECK(2 == inputs.size(), "the Add Function needs 2 input");
}

Shape Add::checkShape(std::vector<Shape> &inputShapes) {
    DEEP8_ARGUMENT_CHECK(2 == inputShapes.size(), "the input count must be 2");
    return broadcastShape(inputShapes[0], inputShapes[1]);
}

ElementType Add::checkElementType(std::vector<ElementType> &inputTypes) {
    DEEP8_ARGUMENT_CHECK(2 == inputTypes.size(), "the input count must be 2");
    return Function::checkElementType(inputTypes);
}

void Add::forward(const std::vector<const Tensor *> &in, Tensor *output) { Math::Add(*in[0], *in[1], *output); }

void Add::backward(const std::vector<const Tensor *> &in, const Tensor *output, const Tensor *outputGradient, size_t index,
                   Tensor *iGradient) {
    if (0 == index) Math::AddGradX(*in[0], *iGradient, *in[1], *output, *outputGradient);
    else if (1 == index) Math::AddGradY(*in[0], *in[1], *iGradient, *output, *outputGradient);
    else DEEP8_RUNTIME_ERROR("the index is error");
}

ReLu::ReLu(std::vector<Node *> &in) : Function(in) {
    DEEP8_ARGUMENT_CHECK(1 == inputs.size(), "the ReLu Function needs 1 input");
}

Shape ReLu::checkShape(std::vector<Shape> &inputShapes) {
    DEEP8_ARGUMENT_CHECK(1 == inputShapes.size(), "the input count must be 1");
    return inputShapes[0];
}

ElementType ReLu::checkElementType(std::vector<ElementType> &inputTypes) {
    DEEP8_ARGUMENT_CHECK(1 == inputTypes.size(), "the input count must be 1");
    return Function::checkElementType(inputTypes);
}

void ReLu::forward(const std::vector<const Tensor *> &in, Tensor *output) { Math::ReLu(*in[0], *output); }

void ReLu::backward(const std::vector<const Tensor *> &in, const Tensor *output, const Tensor *outputGradient, size_t,
                    Tensor *iGradient) {
    Math::ReLuGrad(*in[0], *iGradient, *output, *outputGradient);
}

Minus::Minus(std::vector<Node *> &in) : Function(in) {
    DEEP8_ARGUMENT_CHECK(2 == inputs.size(), "the Minus Function needs 2 input");
}

Shape Minus::checkShape(std::vector<Shape> &inputShapes) {
    DEEP8_ARGUMENT_CHECK(2 == inputShapes.size(), "the input count must be 2");
    return broadcastShape(inputShapes[0], inputShapes[1]);
}

ElementType Minus::checkElementType(std::vector<ElementType> &inputTypes) {
    DEEP8_ARGUMENT_CHECK(2 == inputTypes.size(), "the input count must be 2");
    return Function::checkElementType(inputTypes);
}

void Minus::forward(const std::vector<const Tensor *> &in, Tensor *output) { Math::Minus(*in[0], *in[1], *output); }

void Minus::backward(const std::vector<const Tensor *> &in, const Tensor *output, const Tensor *outputGradient, size_t index,
                     Tensor *iGradient) {
    if (0 == index) Math::MinusGradX(*in[0], *iGradient, *in[1], *output, *outputGradient);
    else if (1 == index) Math::MinusGradY(*in[0], *in[1], *iGradient, *output, *outputGradient);
    else DEEP8_RUNTIME_ERROR("the index is error");
}

L1Norm::L1Norm(std::vector<Node *> &in) : Function(in) {
    DEEP8_ARGUMENT_CHECK(1 == inputs.size(), "the L1Norm Function needs 1 input");
}

Shape L1Norm::checkShape(std::vector<Shape> &inputShapes) {
    DEEP8_ARGUMENT_CHECK(1 == inputShapes.size(), "the input count must be 1");
    return Shape(inputShapes[0].batch, {1});
}

ElementType L1Norm::checkElementType(std::vector<ElementType> &inputTypes) {
    DEEP8_ARGUMENT_CHECK(1 == inputTypes.size(), "the input count must be 1");
    return Function::checkElementType(inputTypes);
}

void L1Norm::forward(const std::vector<const Tensor *> &in, Tensor *output) { Math::L1Norm(*in[0], *output); }

void L1Norm::backward(const std::vector<const Tensor *> &in, const Tensor *output, const Tensor *outputGradient, size_t index,
                      Tensor *iGradient) {
    DEEP8_ARGUMENT_CHECK(0 == index, "the index of L1Norm backward is error");
    Math::L1NormGrad(*in[0], *iGradient, *output, *outputGradient);
}

L2Norm::L2Norm(std::vector<Node *> &in) : Function(in) {
    DEEP8_ARGUMENT_CHECK(1 == inputs.size(), "the L2Norm Function needs 1 input");
}

Shape L2Norm::checkShape(std::vector<Shape> &inputShapes) {
    DEEP8_ARGUMENT_CHECK(1 == inputShapes.size(), "the input count must be 1");
    return Shape(inputShapes[0].batch, {1});
}

ElementType L2Norm::checkElementType(std::vector<ElementType> &inputTypes) {
    DEEP8_ARGUMENT_CHECK(1 == inputTypes.size(), "the input count must be 1");
    return Function::checkElementType(inputTypes);
}

void L2Norm::forward(const std::vector<const Tensor *> &in, Tensor *output) { Math::L2Norm(*in[0], *output); }

void L2Norm::backward(const std::vector<const Tensor *> &in, const Tensor *output, const Tensor *outputGradient, size_t index,
                      Tensor *iGradient) {
    DEEP8_ARGUMENT_CHECK(0 == index, "the index of L2Norm backward is error");
    Math::L2NormGrad(*in[0], *iGradient, *output, *outputGradient);
}

ReduceMean::ReduceMean(std::vector<Node *> &in, std::vector<int> reduceAxis, bool keep)
    : Function(in), axis(reduceAxis), keepDims(keep) {
    DEEP8_ARGUMENT_CHECK(1 == inputs.size(), "the ReduceMean Function needs 1 input");
}

Shape ReduceMean::checkShape(std::vector<Shape> &inputShapes) {
    DEEP8_ARGUMENT_CHECK(1 == inputShapes.size(), "only have 1 input");
    return Math::ReduceMeanShape(inputShapes[0], axis, keepDims);
}

ElementType ReduceMean::checkElementType(std::vector<ElementType> &inputTypes) {
    DEEP8_ARGUMENT_CHECK(1 == inputTypes.size(), "the input count must be 1");
    return Function::checkElementType(inputTypes);
}

void ReduceMean::forward(const std::vector<const Tensor *> &in, Tensor *output) { Math::ReduceMean(*in[0], *output, axis, keepDims); }

void ReduceMean::backward(const std::vector<const Tensor *> &in, const Tensor *output, const Tensor *outputGradient, size_t,
                          Tensor *iGradient) {
    Math::ReduceMeanGrad(*in[0], *iGradient, *output, *outputGradient, axis, keepDims);
}

Pooling2d::Pooling2d(std::vector<Node *> &in, bool mx, bool cov, int fh, int fw, int sy, int sx)
    : Function(in), isMax(mx), covered(cov), filterHeight(fh), filterWidth(fw), strideY(sy), strideX(sx) {
    DEEP8_ARGUMENT_CHECK(1 == inputs.size(), "the pooling Function needs 1 input");
    DEEP8_ARGUMENT_CHECK(fh >= 1 && fw >= 1 && sy >= 1 && sx >= 1, "the filter size or stride is error");
}

Shape Pooling2d::checkShape(std::vector<Shape> &inputShapes) {
    DEEP8_ARGUMENT_CHECK(1 == inputShapes.size(), "the input count must be 1");
    return Math::Pooling2dShape(inputShapes[0], covered, filterHeight, filterWidth, strideY, strideX);
}

ElementType Pooling2d::checkElementType(std::vector<ElementType> &inputTypes) {
    DEEP8_ARGUMENT_CHECK(1 == inputTypes.size(), "the input count must be 1");
    return Function::checkElementType(inputTypes);
}

void Pooling2d::forward(const std::vector<const Tensor *> &in, Tensor *output) {
    if (isMax) Math::MaxPooling2d(*in[0], *output, covered, filterHeight, filterWidth, strideY, strideX);
    else Math::AvgPooling2d(*in[0], *output, covered, filterHeight, filterWidth, strideY, strideX);
}

void Pooling2d::backward(const std::vector<const Tensor *> &in, const Tensor *output, const Tensor *outputGradient, size_t index,
                         Tensor *iGradient) {
    DEEP8_ARGUMENT_CHECK(0 == index, "the index is error");
    if (isMax) Math::MaxPooling2dGrad(*in[0], *iGradient, *output, *outputGradient, covered, filterHeight, filterWidth, strideY, strideX);
    else Math::AvgPooling2dGrad(*in[0], *iGradient, *output, *outputGradient, covered, filterHeight, filterWidth, strideY, strideX);
}

}  // namespace Deep8
