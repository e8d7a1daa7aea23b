#include "tensor.h"
#include "operator.h"

#include <cstring>

namespace tpm {

static pet_hip_stream_t g_stream = nullptr;
static bool g_ready = false;

bool petInit() {
    if (g_ready)
        return true;
    if (!petOk(pet_hip_init(0), "pet_hip_init"))
        return false;
    if (!petOk(pet_hip_stream_create(&g_stream), "pet_hip_stream_create"))
        return false;
    g_ready = true;
    return true;
}

pet_hip_stream_t petStream() {
    petInit();
    return g_stream;
}

Tensor::Tensor(TensorType type, DataType dtype)
    : guid(generateGuid()), hash(generateHash()), dtype(dtype), type(type) {}

Tensor::Tensor(const Dim &dims, TensorType type, DataType dtype)
    : guid(generateGuid()), hash(generateHash()), dims(dims), dtype(dtype), type(type) {}

Tensor::Tensor(const Tensor &rhs)
    : guid(generateGuid()), hash(rhs.hash), dims(rhs.dims), dtype(rhs.dtype), type(rhs.type),
      dimPenalty(rhs.dimPenalty) {}

Tensor::~Tensor() {
    if (dev && ownsDev)
        pet_hip_free(dev);
}

void Tensor::clone(Tensor *t) {
    setDims(t->dims);
    dtype = t->dtype;
    type = t->type;
    hash = t->hash;
    dimPenalty = t->dimPenalty;
}

void Tensor::setDims(const Dim &d) {
    dims = d;
    if (dev && ownsDev && devElems < size()) {
        pet_hip_free(dev);
        dev = nullptr;
        devElems = 0;
        devFresh = false;
    }
    if (host.size() != size()) {
        host.clear();
        hostFresh = false;
    }
}

std::pair<Operator *, int> Tensor::getOutputOfWithIndex() {
    if (!outputOf)
        return {nullptr, -1};
    const auto &outs = outputOf->getOutputs();
    for (size_t i = 0; i < outs.size(); ++i)
        if (outs[i] == this)
            return {outputOf, (int)i};
    return {outputOf, -1};
}

bool Tensor::isClear() const {
    return inputOf.empty() && outputOf == nullptr && type == Input && computed == NotComputed &&
           splittingPoints.empty();
}

void Tensor::clear() {
    inputOf.clear();
    outputOf = nullptr;
    type = Input;
    computed = NotComputed;
    splittingPoints.clear();
    hash = generateHash();
    dimPenalty.clear();
    // a recycled tensor starts without a host mirror (the device buffer stays)
    std::vector<VType>().swap(host);
    hostFresh = false;
}

const Dim &Tensor::getPenalty() {
    if (dimPenalty.size() != dims.size())
        dimPenalty.assign(dims.size(), 0);
    return dimPenalty;
}

Dim Tensor::getPenalty() const {
    return dimPenalty.size() == dims.size() ? dimPenalty : Dim(dims.size(), 0);
}

void Tensor::addPenalty(int d, int penalty) {
    if (dimPenalty.size() != dims.size())
        dimPenalty.assign(dims.size(), 0);
    dimPenalty[d] += penalty;
}

bool Tensor::dataMalloc() {
    if (!petInit())
        return false;
    if (dev && devElems >= size())
        return true;
    if (dev && ownsDev)
        pet_hip_free(dev);
    void *p = nullptr;
    if (!petOk(pet_hip_malloc(&p, std::max<size_t>(size(), 1) * sizeof(float)), "pet_hip_malloc"))
        return false;
    dev = (float *)p;
    devElems = size();
    ownsDev = true;
    devFresh = false;
    return true;
}

// New values in this tensor make everything computed from it stale. The
// reference re-evaluates a requested point from the current inputs every time
// (src/Graph/graph.cc:780-842); here results are kept on the device, so the
// invalidation is explicit.
void Tensor::invalidateDependents() {
    for (auto op : inputOf)
        for (auto out : op->getOutputs())
            if (out != this && out->computed != NotComputed) {
                out->computed = NotComputed;
                out->invalidateDependents();
            }
}

bool Tensor::dataRand(int seed) {
    // one stream of the 214013 / 2531011 generator, reduced to small integers
    // seed 0 (the default) continues one process-wide stream, so that tensors
    // filled one after another differ, as with the reference's persistent
    // generator state; any other seed starts a reproducible stream of its own.
    static int shared = 0;
    host.resize(size());
    int g = seed == 0 ? shared : seed;
    for (size_t i = 0; i < host.size(); ++i) {
        g = (int)(214013u * (unsigned)g + 2531011u);
        host[i] = (VType)(((g >> 16) & 0x7FFF) % kRandMod);
    }
    if (seed == 0)
        shared = g;
    hostFresh = true;
    devFresh = false;
    computed = ComputedFull;
    ++version;
    invalidateDependents();
    return true;
}

bool Tensor::setData(const VType *hostPtr) {
    if (!hostPtr)
        return false;
    host.assign(hostPtr, hostPtr + size());
    hostFresh = true;
    devFresh = false;
    computed = ComputedFull;
    ++version;
    invalidateDependents();
    return true;
}

VType *Tensor::getDataPtr() {
    if (!hostFresh) {
        host.resize(size());
        if (dev && devFresh && size()) {
            pet_hip_stream_sync(petStream());
            petOk(pet_hip_memcpy_d2h(host.data(), dev, size() * sizeof(float), petStream()),
                  "pet_hip_memcpy_d2h");
        }
        hostFresh = true;
    }
    // the caller may write through the pointer: the device copy is stale from now on
    devFresh = false;
    ++version;
    return host.data();
}

float *Tensor::devicePtr() {
    if (!dataMalloc())
        return nullptr;
    if (!devFresh && hostFresh && size()) {
        petOk(pet_hip_memcpy_h2d(dev, host.data(), size() * sizeof(float), petStream()),
              "pet_hip_memcpy_h2d");
    }
    devFresh = true;
    return dev;
}

void Tensor::aliasDevice(float *ptr) {
    ++version;
    if (dev && ownsDev)
        pet_hip_free(dev);
    dev = ptr;
    devElems = size();
    ownsDev = false;
    devFresh = true;
    hostFresh = false;
}

void Tensor::refreshHostMirrorInPlace() {
    if (host.size() != size() || host.empty() || hostFresh || !dev || !devFresh)
        return;
    pet_hip_stream_sync(petStream());
    if (petOk(pet_hip_memcpy_d2h(host.data(), dev, size() * sizeof(float), petStream()),
              "pet_hip_memcpy_d2h"))
        hostFresh = true;
}

void Tensor::deviceWritten() {
    devFresh = true;
    hostFresh = false;
    ++version;
}

size_t Tensor::getOffset(const Dim &pos) const {
    if (pos.size() != dims.size())
        return (size_t)-1;
    size_t off = 0;
    for (size_t i = 0; i < dims.size(); ++i) {
        if (pos[i] < 0 || pos[i] >= dims[i])
            return (size_t)-1;
        off = off * (size_t)dims[i] + (size_t)pos[i];
    }
    return off;
}

bool Tensor::itValid() const {
    if (it.size() != dims.size())
        return false;
    for (size_t i = 0; i < it.size(); ++i)
        if (it[i] >= dims[i])
            return false;
    return true;
}

// Odometer step: the last axis moves fastest; running off the end of axis 0
// leaves it[0] == dims[0], which itValid() reports.
void Tensor::itNext() {
    if (it.empty())
        return;
    size_t p = it.size() - 1;
    ++it[p];
    while (p > 0 && it[p] == dims[p]) {
        it[p] = 0;
        ++it[--p];
    }
}

VType Tensor::getData(const Dim &pos) {
    size_t off = getOffset(pos);
    if (off == (size_t)-1)
        return 0;
    return getData(off);
}

VType Tensor::getData(size_t pos) {
    if (pos >= size())
        return 0;
    bool keepDev = devFresh;
    uint64_t keepVersion = version;
    VType v = getDataPtr()[pos];
    devFresh = keepDev; // a read does not invalidate the device copy
    version = keepVersion;
    return v;
}

bool Tensor::setData(const Dim &pos, VType val) {
    size_t off = getOffset(pos);
    if (off == (size_t)-1)
        return false;
    return setData(off, val);
}

bool Tensor::setData(size_t pos, VType val) {
    if (pos >= size())
        return false;
    getDataPtr()[pos] = val;
    invalidateDependents();
    return true;
}

void Tensor::print() {
    if (type == Invalid) {
        std::cout << "Invalid tensor" << std::endl;
        return;
    }
    if (dims.empty() || size() == 0) {
        std::cout << "Empty tensor" << std::endl;
        return;
    }
    std::cout << "Tensor " << guid << " " << dimToString(dims) << std::endl;
    bool keepDev = devFresh;
    const VType *d = getDataPtr();
    devFresh = keepDev;
    size_t inner = (size_t)dims.back();
    for (size_t i = 0; i < size(); ++i)
        std::cout << d[i] << ((i + 1) % inner == 0 ? "\n" : ", ");
}

void Tensor::printShape() { std::cout << dimToString(dims) << std::endl; }

void printTensor(Tensor *tensor) { tensor->print(); }

} // namespace tpm
