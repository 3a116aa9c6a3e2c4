// Deep8's model core on an MI355X: ElementType, Shape, Device / GPUDevice (+ its buddy memory
// pool), TensorStorage and Tensor.  Names, members and meaning follow the reference so that code
// written against Deep8 compiles against this header:
//   DType / ElementType   deep8/include/model/ElementType.h:8-116
//   Shape                 deep8/include/model/Shape.h:32-83, deep8/src/model/Shape.cpp:86-154
//   Device / GPUDevice    deep8/include/model/Device.h:18-42, deep8/include/model/GPUDevice.h:12-70
//   GPUMemoryPool         deep8/include/model/GPUMemoryPool.h:36-118, deep8/src/model/GPUMemoryPool.cu:132-279
//   TensorStorage         deep8/include/model/TensorStorage.h:13-37
//   Tensor                deep8/include/model/Tensor.h:12-88
// This build carries the GPU path only: DeviceType::CPU exists as a tag, there is no CPUDevice,
// and every Math:: routine refuses CPU tensors instead of falling back.
#ifndef DEEP8_HOST_MODEL_H
#define DEEP8_HOST_MODEL_H

#include <cstddef>
#include <cstdint>
#include <map>
#include <string>
#include <unordered_map>
#include <vector>

#include "deep8/Exception.h"

typedef unsigned char byte;

namespace Deep8 {

// ---------------------------------------------------------------------------------------------
// 16-bit float storage type (the reference uses CUDA's `half` under HAVE_HALF).
struct half {
    uint16_t bits;
    half() : bits(0) {}
    half(float v) : bits(fromFloat(v)) {}
    operator float() const { return toFloat(bits); }
    static uint16_t fromFloat(float v);  // round to nearest even
    static float toFloat(uint16_t h);
};

enum class DType {
    UnKnown = 0, Bool = 1, Uint8 = 2, Int8 = 3, Uint16 = 4, Int16 = 5, Uint32 = 6, Int32 = 7,
    Uint64 = 8, Int64 = 9, Float16 = 10, Float32 = 11, Float64 = 12,
};

class UnKnownType {};

class ElementType {
    ElementType(DType d, size_t bw, std::string n) : id(d), byteWidth(bw), name(std::move(n)) {}

public:
    DType id;
    size_t byteWidth;
    std::string name;

    bool operator==(const ElementType &other) const { return id == other.id; }
    bool operator!=(const ElementType &other) const { return id != other.id; }

    static ElementType unknown() { return ElementType(DType::UnKnown, 0, "unknown"); }
    static ElementType from(DType type);

    template <typename T> static ElementType from();
    template <typename T> bool is() const;
};

template <> inline ElementType ElementType::from<float>() { return from(DType::Float32); }
template <> inline ElementType ElementType::from<double>() { return from(DType::Float64); }
template <> inline ElementType ElementType::from<half>() { return from(DType::Float16); }
template <> inline bool ElementType::is<float>() const { return id == DType::Float32; }
template <> inline bool ElementType::is<double>() const { return id == DType::Float64; }
template <> inline bool ElementType::is<half>() const { return id == DType::Float16; }
template <> inline bool ElementType::is<UnKnownType>() const { return id == DType::UnKnown; }

// ---------------------------------------------------------------------------------------------
#define MAX_TENSOR_DIMS 4

class Shape {
public:
    size_t batch;
    size_t nDims;
    size_t dims[MAX_TENSOR_DIMS];
    size_t strides[MAX_TENSOR_DIMS];

    Shape();
    Shape(const Shape &) = default;
    Shape(size_t batch, const Shape &other);
    explicit Shape(std::vector<size_t> list);
    explicit Shape(size_t batch, std::vector<size_t> list);
    Shape &operator=(const Shape &) = default;

    bool operator==(const Shape &other) const;
    bool operator!=(const Shape &other) const { return !(*this == other); }
    size_t operator[](size_t d) { return dim(d); }

    void reShape(Shape &other);
    bool equalExceptBatch(const Shape &other);

    size_t size() const;       // batch * dims[0] * dims[1] * ...
    size_t batchSize() const;  // size() / batch
    size_t dim(size_t d) const;
    size_t stride(size_t d) const;
    size_t row() const;  // dims[0]
    size_t col() const;  // 1 for a 1-D shape, else dims[1]
    std::string toStr();

private:
    void updateStrides();  // row-major
};

// ---------------------------------------------------------------------------------------------
enum class DeviceType { CPU = 0, GPU = 1 };

class Device {
public:
    DeviceType type;
    explicit Device(DeviceType t) : type(t) {}
    virtual ~Device() = default;

    virtual void *malloc(size_t size) = 0;
    virtual void free(void *ptr) = 0;
    virtual void zero(void *ptr, size_t size) = 0;
    virtual void copy(const void *from, void *to, size_t size) = 0;
    virtual void copyFromCPUToGPU(const void *from, void *to, size_t size) = 0;
    virtual void copyFromGPUToCPU(const void *from, void *to, size_t size) = 0;
    virtual void copyFromGPUToGPU(const void *from, void *to, size_t size) = 0;
    virtual void *mallocCPU(size_t size) = 0;
    virtual void freeCPU(void *ptr) = 0;
    virtual void *gpuOneHalf() = 0;
    virtual void *gpuOneFloat() = 0;
    virtual void *gpuOneDouble() = 0;

    // Deferred zeroing of whole allocations.  The executor zeroes every gradient before a backward
    // pass (deep8/src/model/EagerExecutor.cpp:51-65) and most of them are then written exactly once,
    // by a routine that can just as well overwrite.  zeroLater(ptr, size) records that the
    // allocation starting at ptr reads as zeros from now on; settle(ptr) performs a recorded fill
    // (Tensor::raw() calls it, so every ordinary reader and writer sees real zeros); takeZero(ptr)
    // forgets the record and returns true when there was one -- the caller then owes a full
    // overwrite of the allocation.  free() forgets the record too.
    virtual void zeroLater(void *ptr, size_t size) { zero(ptr, size); }
    virtual void settle(void *) {}
    virtual bool takeZero(void *) { return false; }
};

// Buddy allocator over large hipMalloc'ed blocks.  Requests are rounded up to a power of two and
// served from per-size free lists; a freed chunk is merged with its buddy; blocks go back to the
// driver only when the pool is destroyed, so a pointer freed right after launching kernels on it
// (Deep8's scratch idiom, deep8/src/nodes/Conv2d.cpp:77-82) stays valid for work already queued
// on the same stream.  Chunk metadata lives on the host.
class GPUMemoryPool {
public:
    static const size_t DEFAULT_BLOCK_SIZE = size_t(512) << 20;  // the reference's block size
    static const size_t MIN_CHUNK = 256;

    int deviceId;
    size_t gpuBlockSize;

    explicit GPUMemoryPool(int id = 0, size_t blockSize = DEFAULT_BLOCK_SIZE);
    ~GPUMemoryPool();
    GPUMemoryPool(const GPUMemoryPool &) = delete;
    GPUMemoryPool &operator=(const GPUMemoryPool &) = delete;

    void *malloc(size_t size);  // throws invalid_argument when size > gpuBlockSize
    void free(void *ptr);       // throws runtime_error for a pointer the pool does not own
    void zero(void *ptr, size_t size);
    void copy(const void *from, void *to, size_t size);
    void copyFromCPUToGPU(const void *from, void *to, size_t size);
    void copyFromGPUToCPU(const void *from, void *to, size_t size);
    void copyFromGPUToGPU(const void *from, void *to, size_t size);
    void *mallocCPU(size_t size);
    void freeCPU(void *ptr);

    size_t blockCount() const { return blocks.size(); }
    size_t bytesInUse() const { return inUse; }
    std::string toString();
    void printInfo();

private:
    struct Chunk {
        size_t block;   // index into `blocks`
        size_t offset;  // from the start of the block
        int level;      // chunk size = 1 << level
        bool used;
    };
    int maxLevel;
    size_t inUse;
    std::vector<void *> blocks;
    std::vector<std::map<std::pair<size_t, size_t>, void *>> freeLists;  // per level: (block, offset) -> ptr
    std::unordered_map<void *, Chunk> chunks;                             // every live chunk, free or used
    void addBlock();
};

class GPUDevice : public Device {
public:
    GPUMemoryPool *memoryPool;
    int deviceId;

    double *oneDouble;
    float *oneFloat, *zeroFloat, *minusOneFloat;
    half *oneHalf, *zeroHalf, *minusOneHalf;

    GPUDevice();
    explicit GPUDevice(int id);
    GPUDevice(int id, size_t poolBlockSize);
    ~GPUDevice() override;

    void *malloc(size_t size) override;
    void free(void *ptr) override;
    void *mallocCPU(size_t size) override;
    void freeCPU(void *ptr) override;
    void zero(void *ptr, size_t size) override;
    void copy(const void *from, void *to, size_t size) override;
    void copyFromCPUToGPU(const void *from, void *to, size_t size) override;
    void copyFromGPUToCPU(const void *from, void *to, size_t size) override;
    void copyFromGPUToGPU(const void *from, void *to, size_t size) override;
    void *gpuOneHalf() override;
    void *gpuOneFloat() override;
    void *gpuOneDouble() override;

    void synchronize();  // wait for the default stream (fetch() does this implicitly)

    void zeroLater(void *ptr, size_t size) override;
    void settle(void *ptr) override;
    bool takeZero(void *ptr) override;

private:
    std::unordered_map<void *, size_t> pendingZero;  // allocation -> bytes still to be zeroed
};

// ---------------------------------------------------------------------------------------------
// Reference-counted handle on device memory; the count lives in host memory.
class TensorStorage {
public:
    Device *device;
    void *ptr;
    size_t *refPtr;
    size_t size;

    TensorStorage();
    TensorStorage(void *p, size_t *refP, size_t s, Device *d);
    TensorStorage(const TensorStorage &other);
    ~TensorStorage();
    TensorStorage &operator=(const TensorStorage &other);

protected:
    void release();
};

class Tensor {
public:
    TensorStorage storage;
    size_t offset;  // bytes into storage
    Shape shape;
    ElementType elementType;

    Tensor();
    explicit Tensor(Shape &s);
    Tensor(TensorStorage &ts, size_t off, Shape &s, ElementType et);
    Tensor(TensorStorage &ts, size_t off, std::vector<size_t> &list, ElementType et);
    Tensor(TensorStorage &ts, size_t off, size_t batch, std::vector<size_t> &list, ElementType et);

    DeviceType deviceType() const { return storage.device->type; }
    Device *device() const { return storage.device; }
    size_t *refPtr() const { return storage.refPtr; }
    size_t refCount() const { return storage.refPtr[0]; }
    // Device address of the first element; performs a deferred zero fill of the allocation first.
    void *raw() const {
        if (storage.device) storage.device->settle(storage.ptr);
        return (byte *)storage.ptr + offset;
    }
    // For a routine that is about to write every element: true when the tensor is a whole
    // allocation whose zero fill was still deferred (the fill is dropped: write, do not add);
    // otherwise false, with any deferred fill performed.
    bool takeZero() const {
        if (!storage.device) return false;
        if (0 == offset && byteCount() == storage.size) return storage.device->takeZero(storage.ptr);
        storage.device->settle(storage.ptr);
        return false;
    }

    bool isScalar() const { return 1 == shape.size(); }
    void zero();
    void one();

    size_t byteCount() const { return elementType.byteWidth * shape.size(); }
    size_t batch() const { return shape.batch; }
    size_t nDims() const { return shape.nDims; }
    size_t size() const { return shape.size(); }
    size_t batchSize() const { return shape.batchSize(); }
    size_t row() const { return shape.row(); }
    size_t col() const { return shape.col(); }
    size_t dim(size_t d) const { return shape.dim(d); }
    size_t stride(size_t d) const { return shape.stride(d); }
    std::string valueStr();

    template <typename T>
    T *data() const {
        DEEP8_ARGUMENT_CHECK(elementType.is<T>(), "Tensor type is error, type is: " << elementType.name);
        return (T *)raw();
    }
    template <typename T>
    bool is() const { return elementType.is<T>(); }
};

}  // namespace Deep8

#endif
