// ElementType, Shape, GPUMemoryPool, GPUDevice, TensorStorage and Tensor (see deep8/Model.h).
#include "deep8/Model.h"

#include <cstring>
#include <iostream>

#include "deep8_hip.h"

namespace Deep8 {

// ---- half <-> float (round to nearest even) -------------------------------------------------------
uint16_t half::fromFloat(float v) {
    uint32_t x;
    std::memcpy(&x, &v, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t mag = x & 0x7fffffffu;
    if (mag >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (mag > 0x7f800000u ? 0x200u : 0));  // inf / nan
    if (mag >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);                                      // overflow
    if (mag < 0x38800000u) {  // subnormal half or zero
        if (mag < 0x33000000u) return (uint16_t)sign;
        const int shift = 113 - (int)(mag >> 23);
        const uint32_t man = (mag & 0x7fffffu) | 0x800000u;
        uint32_t h = man >> (shift + 13);
        const uint32_t rem = man & ((1u << (shift + 13)) - 1), halfway = 1u << (shift + 12);
        if (rem > halfway || (rem == halfway && (h & 1))) ++h;
        return (uint16_t)(sign | h);
    }
    uint32_t h = ((mag - 0x38000000u) >> 13);
    const uint32_t rem = mag & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1))) ++h;
    return (uint16_t)(sign | h);
}

float half::toFloat(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f, man = h & 0x3ffu, x;
    if (exp == 0) {
        if (man == 0) {
            x = sign;
        } else {
            int e = -1;
            do {
                ++e;
                man <<= 1;
            } while (!(man & 0x400u));
            x = sign | ((uint32_t)(112 - e) << 23) | ((man & 0x3ffu) << 13);
        }
    } else if (exp == 31) {
        x = sign | 0x7f800000u | (man << 13);
    } else {
        x = sign | ((exp + 112) << 23) | (man << 13);
    }
    float f;
    std::memcpy(&f, &x, 4);
    return f;
}

// ---- ElementType -------------------------------------------------------------------------------------
ElementType ElementType::from(DType type) {
    switch (type) {
    case DType::UnKnown: return ElementType(DType::UnKnown, 0, "unknown");
    case DType::Bool: return ElementType(DType::Bool, sizeof(bool), "bool");
    case DType::Uint8: return ElementType(DType::Uint8, 1, "uint8_t");
    case DType::Int8: return ElementType(DType::Int8, 1, "int8_t");
    case DType::Uint16: return ElementType(DType::Uint16, 2, "uint16_t");
    case DType::Int16: return ElementType(DType::Int16, 2, "int16_t");
    case DType::Uint32: return ElementType(DType::Uint32, 4, "uint32_t");
    case DType::Int32: return ElementType(DType::Int32, 4, "int32_t");
    case DType::Uint64: return ElementType(DType::Uint64, 8, "uint64_t");
    case DType::Int64: return ElementType(DType::Int64, 8, "int64_t");
    case DType::Float16: return ElementType(DType::Float16, 2, "float16");
    case DType::Float32: return ElementType(DType::Float32, 4, "float32");
    case DType::Float64: return ElementType(DType::Float64, 8, "float64");
    }
    DEEP8_RUNTIME_ERROR("the dtype is error");
}

// ---- Shape -----------------------------------------------------------------------------------------------
Shape::Shape() : batch(0), nDims(0), dims{0}, strides{0} {}

Shape::Shape(size_t b, const Shape &other) : Shape(other) { batch = b; }

Shape::Shape(std::vector<size_t> list) : Shape(1, std::move(list)) {}

Shape::Shape(size_t b, std::vector<size_t> list) : batch(b), nDims(0), dims{0}, strides{0} {
    DEEP8_ARGUMENT_CHECK(1 <= list.size() && list.size() <= MAX_TENSOR_DIMS,
                         "the list size:" << list.size() << " is error must >= 1 and <= " << MAX_TENSOR_DIMS);
    for (size_t d : list) {
        DEEP8_ARGUMENT_CHECK(0 != d, "the dim can not be 0");
        dims[nDims++] = d;
    }
    updateStrides();
}

void Shape::updateStrides() {
    size_t running = 1;
    for (size_t i = nDims; i-- > 0;) {
        strides[i] = running;
        running *= dims[i];
    }
}

bool Shape::operator==(const Shape &other) const {
    if (batch != other.batch || nDims != other.nDims) return false;
    for (size_t i = 0; i < nDims; ++i)
        if (dims[i] != other.dims[i]) return false;
    return true;
}

bool Shape::equalExceptBatch(const Shape &other) {
    if (nDims != other.nDims) return false;
    for (size_t i = 0; i < nDims; ++i)
        if (dims[i] != other.dims[i]) return false;
    return true;
}

void Shape::reShape(Shape &other) {
    DEEP8_ARGUMENT_CHECK(size() == other.size(), "the reShape operator needs this 2 Shape have the same size");
    *this = other;
}

size_t Shape::size() const { return 0 == nDims ? 0 : batch * batchSize(); }
size_t Shape::batchSize() const { return 0 == nDims ? 0 : dims[0] * strides[0]; }

size_t Shape::dim(size_t d) const {
    DEEP8_ARGUMENT_CHECK(d < nDims, "the Tensor does't have dimensions " << d);
    return dims[d];
}

size_t Shape::stride(size_t d) const {
    DEEP8_ARGUMENT_CHECK(d < nDims, "the Tensor does't have dimensions " << d);
    return strides[d];
}

size_t Shape::row() const {
    DEEP8_ARGUMENT_CHECK(nDims >= 1, "the dimensions is error");
    return dims[0];
}

size_t Shape::col() const {
    DEEP8_ARGUMENT_CHECK(nDims >= 1, "the dimensions is error");
    return 1 == nDims ? 1 : dims[1];
}

std::string Shape::toStr() {
    std::ostringstream out;
    out << "[" << batch;
    for (size_t i = 0; i < nDims; ++i) out << ", " << dims[i];
    out << "]";
    return out.str();
}

// ---- GPUMemoryPool -----------------------------------------------------------------------------------------
static int levelOf(size_t size) {  // smallest L with (1 << L) >= size
    int level = 0;
    while ((size_t(1) << level) < size) ++level;
    return level;
}

GPUMemoryPool::GPUMemoryPool(int id, size_t blockSize) : deviceId(id), gpuBlockSize(blockSize), inUse(0) {
    DEEP8_ARGUMENT_CHECK(blockSize >= MIN_CHUNK && 0 == (blockSize & (blockSize - 1)),
                         "the memory block size must be a power of 2");
    maxLevel = levelOf(blockSize);
    freeLists.resize(maxLevel + 1);
}

GPUMemoryPool::~GPUMemoryPool() {
    for (void *block : blocks) d8_free(block);
}

void GPUMemoryPool::addBlock() {
    void *ptr = nullptr;
    D8_CHECK(d8_malloc(&ptr, gpuBlockSize));
    blocks.push_back(ptr);
    chunks[ptr] = Chunk{blocks.size() - 1, 0, maxLevel, false};
    freeLists[maxLevel][{blocks.size() - 1, 0}] = ptr;
}

void *GPUMemoryPool::malloc(size_t size) {
    if (0 == size) return nullptr;
    DEEP8_ARGUMENT_CHECK(size <= gpuBlockSize, "malloc too much memory");
    const int want = levelOf(size < MIN_CHUNK ? MIN_CHUNK : size);

    int level = want;
    while (level <= maxLevel && freeLists[level].empty()) ++level;
    if (level > maxLevel) {
        addBlock();
        level = maxLevel;
    }
    // take the lowest-addressed free chunk of that level and halve it down to the wanted size
    auto it = freeLists[level].begin();
    void *ptr = it->second;
    freeLists[level].erase(it);
    Chunk chunk = chunks[ptr];
    while (chunk.level > want) {
        --chunk.level;
        const size_t halfSize = size_t(1) << chunk.level;
        void *right = (byte *)ptr + halfSize;
        chunks[right] = Chunk{chunk.block, chunk.offset + halfSize, chunk.level, false};
        freeLists[chunk.level][{chunk.block, chunk.offset + halfSize}] = right;
    }
    chunk.used = true;
    chunks[ptr] = chunk;
    inUse += size_t(1) << chunk.level;
    return ptr;
}

void GPUMemoryPool::free(void *ptr) {
    if (nullptr == ptr) return;
    auto found = chunks.find(ptr);
    if (found == chunks.end() || !found->second.used) DEEP8_RUNTIME_ERROR("free memory error");
    Chunk chunk = found->second;
    inUse -= size_t(1) << chunk.level;
    chunks.erase(found);
    // merge with the buddy while it is free and of the same size
    while (chunk.level < maxLevel) {
        const size_t sz = size_t(1) << chunk.level;
        const size_t buddyOffset = chunk.offset ^ sz;
        auto &list = freeLists[chunk.level];
        auto buddy = list.find({chunk.block, buddyOffset});
        if (buddy == list.end()) break;
        chunks.erase(buddy->second);
        list.erase(buddy);
        chunk.offset &= ~sz;
        ++chunk.level;
    }
    chunk.used = false;
    void *merged = (byte *)blocks[chunk.block] + chunk.offset;
    chunks[merged] = chunk;
    freeLists[chunk.level][{chunk.block, chunk.offset}] = merged;
}

void GPUMemoryPool::zero(void *ptr, size_t size) { D8_CHECK(d8_memset(ptr, 0, size, nullptr)); }
void GPUMemoryPool::copy(const void *from, void *to, size_t size) { copyFromGPUToGPU(from, to, size); }
void GPUMemoryPool::copyFromCPUToGPU(const void *from, void *to, size_t size) { D8_CHECK(d8_memcpy_h2d(to, from, size)); }
void GPUMemoryPool::copyFromGPUToCPU(const void *from, void *to, size_t size) { D8_CHECK(d8_memcpy_d2h(to, from, size)); }
void GPUMemoryPool::copyFromGPUToGPU(const void *from, void *to, size_t size) { D8_CHECK(d8_memcpy_d2d(to, from, size, nullptr)); }

void *GPUMemoryPool::mallocCPU(size_t size) {
    void *p = ::operator new(size);
    return p;
}

void GPUMemoryPool::freeCPU(void *ptr) { ::operator delete(ptr); }

std::string GPUMemoryPool::toString() {
    std::ostringstream out;
    out << "GPUMemoryPool(device " << deviceId << "): " << blocks.size() << " block(s) of " << gpuBlockSize
        << " bytes, " << inUse << " bytes in use;";
    for (int level = 0; level <= maxLevel; ++level)
        if (!freeLists[level].empty()) out << " free[2^" << level << "]=" << freeLists[level].size();
    return out.str();
}

void GPUMemoryPool::printInfo() { std::cout << toString() << std::endl; }

// ---- GPUDevice -------------------------------------------------------------------------------------------------
GPUDevice::GPUDevice() : GPUDevice(0) {}

GPUDevice::GPUDevice(int id) : GPUDevice(id, GPUMemoryPool::DEFAULT_BLOCK_SIZE) {}

GPUDevice::GPUDevice(int id, size_t poolBlockSize) : Device(DeviceType::GPU), memoryPool(nullptr), deviceId(id) {
    D8_CHECK(d8_device_init(deviceId));
    memoryPool = new GPUMemoryPool(deviceId, poolBlockSize);

    // {1, 0, -1} in double, float and half, one pool allocation (the reference keeps the same constants)
    void *ptr = memoryPool->malloc(sizeof(double) * 3 + sizeof(float) * 3 + sizeof(half) * 3);
    oneDouble = (double *)ptr;
    oneFloat = (float *)(oneDouble + 3);
    zeroFloat = oneFloat + 1;
    minusOneFloat = zeroFloat + 1;
    oneHalf = (half *)(minusOneFloat + 1);
    zeroHalf = oneHalf + 1;
    minusOneHalf = zeroHalf + 1;
    const float numberF[3] = {1.f, 0.f, -1.f};
    const half numberH[3] = {half(1.f), half(0.f), half(-1.f)};
    const double numberD[3] = {1., 0., -1.};
    memoryPool->copyFromCPUToGPU(numberD, oneDouble, sizeof(numberD));
    memoryPool->copyFromCPUToGPU(numberF, oneFloat, sizeof(numberF));
    memoryPool->copyFromCPUToGPU(numberH, oneHalf, sizeof(numberH));
}

GPUDevice::~GPUDevice() {
    d8_stream_sync(nullptr);
    memoryPool->free(oneDouble);
    delete memoryPool;
}

void *GPUDevice::malloc(size_t size) { return memoryPool->malloc(size); }
void GPUDevice::free(void *ptr) {
    pendingZero.erase(ptr);
    memoryPool->free(ptr);
}
void *GPUDevice::mallocCPU(size_t size) { return memoryPool->mallocCPU(size); }
void GPUDevice::freeCPU(void *ptr) { memoryPool->freeCPU(ptr); }
void GPUDevice::zero(void *ptr, size_t size) { memoryPool->zero(ptr, size); }
void GPUDevice::copy(const void *from, void *to, size_t size) { memoryPool->copy(from, to, size); }
void GPUDevice::copyFromCPUToGPU(const void *from, void *to, size_t size) { memoryPool->copyFromCPUToGPU(from, to, size); }
void GPUDevice::copyFromGPUToCPU(const void *from, void *to, size_t size) { memoryPool->copyFromGPUToCPU(from, to, size); }
void GPUDevice::copyFromGPUToGPU(const void *from, void *to, size_t size) { memoryPool->copyFromGPUToGPU(from, to, size); }
void *GPUDevice::gpuOneHalf() { return oneHalf; }
void *GPUDevice::gpuOneFloat() { return oneFloat; }
void *GPUDevice::gpuOneDouble() { return oneDouble; }
void GPUDevice::synchronize() { D8_CHECK(d8_stream_sync(nullptr)); }

void GPUDevice::zeroLater(void *ptr, size_t size) { pendingZero[ptr] = size; }

void GPUDevice::settle(void *ptr) {
    if (pendingZero.empty()) return;
    auto it = pendingZero.find(ptr);
    if (it == pendingZero.end()) return;
    const size_t size = it->second;
    pendingZero.erase(it);
    zero(ptr, size);
}

bool GPUDevice::takeZero(void *ptr) { return !pendingZero.empty() && pendingZero.erase(ptr) > 0; }

// ---- TensorStorage ---------------------------------------------------------------------------------------------------
TensorStorage::TensorStorage() : device(nullptr), ptr(nullptr), refPtr(nullptr), size(0) {}

TensorStorage::TensorStorage(void *p, size_t *refP, size_t s, Device *d) : device(d), ptr(p), refPtr(refP), size(s) {
    DEEP8_ARGUMENT_CHECK(nullptr != p && nullptr != refP && s > 0 && nullptr != d, "the memory is error");
    *refPtr = 1;
}

TensorStorage::TensorStorage(const TensorStorage &other)
    : device(other.device), ptr(other.ptr), refPtr(other.refPtr), size(other.size) {
    if (refPtr) ++*refPtr;
}

TensorStorage::~TensorStorage() { release(); }

TensorStorage &TensorStorage::operator=(const TensorStorage &other) {
    if (other.refPtr) ++*other.refPtr;
    release();
    device = other.device;
    ptr = other.ptr;
    refPtr = other.refPtr;
    size = other.size;
    return *this;
}

void TensorStorage::release() {
    if (refPtr && 0 == --*refPtr) {
        DEEP8_ASSERT(DeviceType::GPU == device->type, "only GPU storage exists in this build");
        device->free(ptr);
        device->freeCPU(refPtr);
    }
    device = nullptr;
    ptr = nullptr;
    refPtr = nullptr;
    size = 0;
}

// ---- Tensor ----------------------------------------------------------------------------------------------------------------
Tensor::Tensor() : storage(), offset(0), shape(), elementType(ElementType::unknown()) {}
Tensor::Tensor(Shape &s) : storage(), offset(0), shape(s), elementType(ElementType::unknown()) {}
Tensor::Tensor(TensorStorage &ts, size_t off, Shape &s, ElementType et) : storage(ts), offset(off), shape(s), elementType(et) {}
Tensor::Tensor(TensorStorage &ts, size_t off, std::vector<size_t> &list, ElementType et) : Tensor(ts, off, 1, list, et) {}
Tensor::Tensor(TensorStorage &ts, size_t off, size_t batch, std::vector<size_t> &list, ElementType et)
    : storage(ts), offset(off), shape(batch, list), elementType(et) {}

void Tensor::zero() { storage.device->zero(raw(), byteCount()); }

void Tensor::one() {
    DEEP8_ARGUMENT_CHECK(isScalar(), "the tensor is not a scalar");
    Device *dev = device();
    switch (elementType.id) {
    case DType::Float64: dev->copyFromGPUToGPU(dev->gpuOneDouble(), raw(), elementType.byteWidth); break;
    case DType::Float32: dev->copyFromGPUToGPU(dev->gpuOneFloat(), raw(), elementType.byteWidth); break;
    case DType::Float16: dev->copyFromGPUToGPU(dev->gpuOneHalf(), raw(), elementType.byteWidth); break;
    default: DEEP8_RUNTIME_ERROR("the type is not support");
    }
}

std::string Tensor::valueStr() {
    std::vector<byte> host(byteCount());
    device()->copyFromGPUToCPU(raw(), host.data(), host.size());
    std::ostringstream out;
    out << "[";
    for (size_t i = 0; i < size(); ++i) {
        if (i) out << ", ";
        if (elementType.id == DType::Float64) out << ((double *)host.data())[i];
        else if (elementType.id == DType::Float32) out << ((float *)host.data())[i];
        else if (elementType.id == DType::Float16) out << (float)((half *)host.data())[i];
        else DEEP8_RUNTIME_ERROR("the type is not support");
    }
    out << "]";
    return out.str();
}

}  // namespace Deep8
