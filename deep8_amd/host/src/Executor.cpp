// Executor, EagerExecutor and the Net.h sugar of the path (see deep8/Executor.h).
#include "deep8/Executor.h"

#include <functional>
#include <queue>

namespace Deep8 {

Executor::Executor(DeviceType deviceType) : uniqueId(0), device(nullptr) {
    if (DeviceType::GPU != deviceType)
        DEEP8_RUNTIME_ERROR("this build carries the GPU path only: a CPU executor can not be created");
    initDeviceGPU();
}

Executor::~Executor() {
    for (auto &item : allNodes) delete item.second;
    allNodes.clear();
    retainVariables.clear();
    interimNodes.clear();
    delete device;
}

void Executor::initDeviceGPU() { device = new GPUDevice(); }

std::string Executor::namePrefix(NameType nameType) {
    switch (nameType) {
    case NameType::Node: return "Node_";
    case NameType::Variable: return "Variable_";
    case NameType::Function: return "Function_";
    case NameType::Conv2d_Weight: return "Conv2d_Weight_";
    case NameType::Conv2d_Bias: return "Conv2d_Bias_";
    case NameType::DeConv2d_Weight: return "DeConv2d_Weight_";
    case NameType::DeConv2d_Bias: return "DeConv2d_Bias_";
    case NameType::MatrixMultiply_Weight: return "MatrixMultiply_Weight_";
    }
    DEEP8_RUNTIME_ERROR("the name type is error");
}

std::string Executor::generateUniqueName(NameType nameType) {
    const std::string prefix = namePrefix(nameType);
    std::string name;
    do {
        name = prefix + std::to_string(nameUniqueId[prefix]++);
    } while (uniqueNames.count(name));
    uniqueNames.insert(name);
    return name;
}

int64_t Executor::generateUniqueId() { return uniqueId++; }

Tensor Executor::createTensor(Shape &shape, DType type) { return createTensor(shape, ElementType::from(type)); }
Tensor Executor::createTensor(Shape &shape, ElementType type) { return createTensorGPU(shape, type); }

// data from the device pool, reference count in host memory
Tensor Executor::createTensorGPU(Shape &shape, ElementType type) {
    const size_t bytes = type.byteWidth * shape.size();
    void *ptr = device->malloc(bytes);
    size_t *refPtr = (size_t *)device->mallocCPU(sizeof(size_t));
    TensorStorage storage(ptr, refPtr, bytes, device);
    return Tensor(storage, 0, shape, type);
}

Variable *Executor::createVariableByFunction(Function *func) {
    const int64_t id = generateUniqueId();
    const std::string name = generateUniqueName(NameType::Variable);
    if (func->isShared()) return new Variable(id, name, this, func);

    bool wantsGradient = false;
    std::vector<Shape> shapes;
    std::vector<ElementType> types;
    for (Node *n : func->inputs) {
        DEEP8_ARGUMENT_CHECK(NodeType::Variable == n->type, "the input must be a Variable");
        Variable *in = (Variable *)n;
        shapes.push_back(in->shape());
        types.push_back(in->elementType());
        wantsGradient = wantsGradient || in->updateGradient;
    }
    Shape shape = func->checkShape(shapes);
    ElementType type = func->checkElementType(types);
    Tensor value = createTensor(shape, type);
    if (!wantsGradient) return new Variable(id, name, this, func, value);
    Tensor gradient = createTensor(shape, type);
    return new Variable(id, name, this, func, value, gradient);
}

void Executor::clearInterimNodes() {
    for (auto &item : allNodes) {
        item.second->inputs.clear();
        item.second->outputs.clear();
    }
    for (auto &item : interimNodes) {
        allNodes.erase(item.first);
        retainVariables.erase(item.first);
        delete item.second;
    }
    interimNodes.clear();
}

void Executor::removeGradient() {
    for (auto &item : allNodes)
        if (NodeType::Variable == item.second->type) ((Variable *)item.second)->removeGradient();
}

Variable *Executor::addVariable(Shape &shape, ElementType type, bool updateGradient, bool retain) {
    return addVariable(shape, type.id, updateGradient, retain);
}
Variable *Executor::addVariable(std::vector<size_t> list, ElementType type, bool updateGradient, bool retain) {
    return addVariable(list, type.id, updateGradient, retain);
}
Variable *Executor::addVariable(size_t batch, std::vector<size_t> list, ElementType type, bool updateGradient, bool retain) {
    return addVariable(batch, list, type.id, updateGradient, retain);
}
Variable *Executor::addVariable(std::vector<size_t> list, DType type, bool updateGradient, bool retain) {
    Shape shape(list);
    return addVariable(shape, type, updateGradient, retain);
}
Variable *Executor::addVariable(size_t batch, std::vector<size_t> list, DType type, bool updateGradient, bool retain) {
    Shape shape(batch, list);
    return addVariable(shape, type, updateGradient, retain);
}
Variable *Executor::addVariable(Shape &shape, DType type, bool updateGradient, bool retain) {
    return addVariable(generateUniqueName(NameType::Variable), shape, type, updateGradient, retain);
}
Variable *Executor::addVariable(std::string name, size_t batch, std::vector<size_t> list, DType type, bool updateGradient, bool retain) {
    Shape shape(batch, list);
    return addVariable(name, shape, type, updateGradient, retain);
}

Variable *Executor::addVariable(std::string name, Shape &shape, DType type, bool updateGradient, bool retain) {
    DEEP8_ARGUMENT_CHECK(!allNodes.count(name), "The name:" << name << "have been used, should set a uniqe name");
    uniqueNames.insert(name);
    const int64_t id = generateUniqueId();
    Tensor value = createTensor(shape, type);
    Variable *variable;
    if (updateGradient) {
        Tensor gradient = createTensor(shape, type);
        variable = new Variable(id, name, this, value, gradient);
    } else {
        variable = new Variable(id, name, this, value);
    }
    allNodes[name] = variable;
    if (retain) retainVariables[name] = variable;
    else interimNodes[name] = variable;
    return variable;
}

Node *Executor::nodeByName(std::string name) {
    auto it = allNodes.find(name);
    return it == allNodes.end() ? nullptr : it->second;
}

Variable *Executor::retainVariableByName(std::string name) {
    auto it = retainVariables.find(name);
    return it == retainVariables.end() ? nullptr : it->second;
}

std::vector<Variable *> Executor::trainableParameters() {
    std::vector<Variable *> out;
    for (auto &item : retainVariables)
        if (item.second->updateGradient) out.push_back(item.second);
    return out;
}

Variable *Executor::addFunction(Function *) { DEEP8_RUNTIME_ERROR("Can not call this function from Executor"); }
void Executor::forward(Node *) { DEEP8_RUNTIME_ERROR("Can not call this function from Executor"); }
void Executor::backward(Node *, bool) { DEEP8_RUNTIME_ERROR("Can not call this function from Executor"); }

// ---- EagerExecutor ---------------------------------------------------------------------------------------------
EagerExecutor::EagerExecutor(DeviceType deviceType) : Executor(deviceType) {}

// The function runs at once: its output Variable is created from checkShape/checkElementType and
// forward() fills it.
Variable *EagerExecutor::addFunction(Function *function) {
    function->id = generateUniqueId();
    function->name = generateUniqueName(NameType::Function);
    function->executor = this;
    Variable *variable = createVariableByFunction(function);
    allNodes[function->name] = function;
    allNodes[variable->name] = variable;
    interimNodes[function->name] = function;
    interimNodes[variable->name] = variable;
    function->forward();
    return variable;
}

void EagerExecutor::forward(Node *) { DEEP8_RUNTIME_ERROR("the EagerExecutor can not call the forward"); }

// Breadth-first from `last` over node->inputs, twice: zero every gradient, then call backward()
// on every node in the same order.
static void breadthFirst(Node *last, const std::function<void(Node *)> &visit) {
    std::queue<Node *> queue;
    std::unordered_set<Node *> seen;
    queue.push(last);
    seen.insert(last);
    while (!queue.empty()) {
        Node *node = queue.front();
        queue.pop();
        visit(node);
        for (Node *input : node->inputs)
            if (seen.insert(input).second) queue.push(input);
    }
}

void EagerExecutor::backward(Node *last, bool clearInterim) {
    DEEP8_ARGUMENT_CHECK(nullptr != last && NodeType::Variable == last->type, "the last node must be a Variable");
    Variable *lastVariable = (Variable *)last;
    DEEP8_ARGUMENT_CHECK(lastVariable->isScalar(), "the last Variable gradient must be scalar");

    breadthFirst(last, [](Node *node) {
        if (NodeType::Variable == node->type && ((Variable *)node)->updateGradient) ((Variable *)node)->zeroGradient();
    });
    lastVariable->oneGradient();
    breadthFirst(last, [](Node *node) { node->backward(); });
    if (clearInterim) clearInterimNodes();
}

// ---- Net sugar ---------------------------------------------------------------------------------------------------------
void backward(Variable &v, bool clearInterim) { v.executor->backward(&v, clearInterim); }
void backward(Variable *v, bool clearInterim) { v->executor->backward(v, clearInterim); }

Variable &parameter(Executor *executor, std::vector<size_t> list, bool updateGradient, DType type) {
    return *executor->addVariable(list, type, updateGradient);
}
Variable &parameter(Executor *executor, size_t batch, std::vector<size_t> list, bool updateGradient, DType type) {
    return *executor->addVariable(batch, list, type, updateGradient);
}
Variable &inputParameter(Executor *executor, std::vector<size_t> list, DType type) {
    return *executor->addVariable(list, type, false, false);
}
Variable &inputParameter(Executor *executor, size_t batch, std::vector<size_t> list, DType type) {
    return *executor->addVariable(batch, list, type, false, false);
}
Variable &feed(Variable &v, const void *ptr) { return v.feed(ptr); }
Variable &fetch(Variable &v, void *ptr) { return v.fetch(ptr); }
Variable &operator*(Variable &x, Variable &y) { return x.matrixMultiply(y); }
Variable &matrixMultiply(Variable &x, Variable &y) { return x.matrixMultiply(y); }
Variable &conv2d(Variable &x, Variable &filter, bool covered, int strideY, int strideX, int dilationY, int dilationX) {
    return x.conv2d(filter, covered, strideY, strideX, dilationY, dilationX);
}
Variable &deConv2d(Variable &x, Variable &filter, bool covered, int strideY, int strideX) {
    return x.deConv2d(filter, covered, strideY, strideX);
}

Variable &operator+(Variable &x, Variable &y) { return x.add(y); }
Variable &add(Variable &x, Variable &y) { return x.add(y); }
Variable &operator-(Variable &x, Variable &y) { return x.minus(y); }
Variable &minus(Variable &x, Variable &y) { return x.minus(y); }
Variable &l1Norm(Variable &x) { return x.l1Norm(); }
Variable &l2Norm(Variable &x) { return x.l2Norm(); }
Variable &reduceMean(Variable &x, std::vector<int> axis, bool keepDims) { return x.reduceMean(axis, keepDims); }
Variable &l1NormLoss(Variable &x) { return x.l1NormLoss(); }
Variable &l2NormLoss(Variable &x) { return x.l2NormLoss(); }
Variable &relu(Variable &x) { return x.relu(); }
Variable &matrixMultiplyBiasReLu(Variable &x, Variable &y, Variable &bias) { return x.matrixMultiplyBiasReLu(y, bias); }
Variable &conv2dBiasReLu(Variable &x, Variable &filter, Variable &bias, bool covered, int strideY, int strideX, int dilationY, int dilationX) {
    return x.conv2dBiasReLu(filter, bias, covered, strideY, strideX, dilationY, dilationX);
}

}  // namespace Deep8
