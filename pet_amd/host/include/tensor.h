// Tensor of the PET graph on the MI355X backend (role of the reference's
// include/tensor.h). The authoritative copy lives in HBM; a host mirror is kept
// for the accessors the mutators and tests use (getData / setData / getDataPtr)
// and is synchronised lazily in whichever direction is stale.
#pragma once
#include "common.h"
#include "dim.h"

namespace tpm {

class Tensor {
  public:
    enum DataType { Float32, Int32 };
    enum TensorType { Input, Weight, Invalid, NotCounted };
    enum ComputeState { NotComputed, ComputedFull };

    Tensor(TensorType type = Input, DataType dtype = Float32);
    Tensor(const Dim &dims, TensorType type = Input, DataType dtype = Float32);
    Tensor(const Tensor &rhs); // shape / type / hash / penalty; no data, no connections
    ~Tensor();
    Tensor &operator=(const Tensor &) = delete;

    Tensor *clone() { return new Tensor(*this); }
    void clone(Tensor *t);

    DataType getDType() const { return dtype; }
    size_t getGuid() const { return guid; }
    uint64_t getHash() const { return hash; }
    void replace(Tensor &t) { hash = t.hash; }
    void refresh() { hash = generateHash(); }

    const Dim &getDims() const { return dims; }
    void setDims(const Dim &d);
    size_t size() const { return dimProduct(dims); }
    bool isScalar() const { return dims.empty(); }

    TensorType getType() const { return type; }
    void setType(TensorType t) { type = t; }
    bool isValid() const { return type != Invalid; }
    void setInvalid() { type = Invalid; }
    bool isNotCounted() const { return type == NotCounted; }

    // graph wiring
    void setInputOf(const OpVec &v) { inputOf = v; }
    void addInputOf(Operator *op) { inputOf.push_back(op); }
    void setOutputOf(Operator *op) { outputOf = op; }
    const OpVec &getInputOf() { return inputOf; }
    Operator *getOutputOf() { return outputOf; }
    std::pair<Operator *, int> getOutputOfWithIndex();
    bool isClear() const;
    void clear();

    bool isComputed() const { return computed == ComputedFull; }
    void setComputed() { computed = ComputedFull; }
    void setNotComputed() { computed = NotComputed; }

    // boundary-correction penalty (extra rows a transformed program carries)
    void resetPenalty() { dimPenalty.assign(dims.size(), 0); }
    const Dim &getPenalty();
    Dim getPenalty() const;
    void addPenalty(int d, int penalty = 1);
    void setPenalty(const Dim &p) { dimPenalty = p; }

    // ---- data ---------------------------------------------------------------
    // Allocates the device buffer (idempotent).
    bool dataMalloc();
    // Fills with the reference's LCG stream (include/tensor.h:371-374), one
    // thread's worth, reduced modulo `kRandMod` so that fp32 contractions of
    // the values stay exact (the reference uses % 10000 in uint32). Seed 0
    // continues a process-wide stream; other seeds are reproducible streams.
    bool dataRand(int seed = 0);
    static constexpr int kRandMod = 8;
    // Copies size() values from a host array to the device.
    bool setData(const VType *hostPtr);
    bool setData(const Dim &pos, VType val);
    bool setData(size_t pos, VType val);
    VType getData(const Dim &pos); // 0 outside the tensor, like the reference
    VType getData(size_t pos);
    VType getBroadcastData(size_t pos) { return getData(pos % size()); }
    // Host mirror, refreshed from the device when stale. Writing through the
    // pointer makes the host copy authoritative until the next device use.
    VType *getDataPtr();
    // Device pointer, refreshed from the host mirror when that is newer.
    float *devicePtr();
    // Adopts device memory owned elsewhere (zero-copy split / concat on dim 0).
    void aliasDevice(float *ptr);
    // Marks the device copy as just written by a kernel.
    void deviceWritten();
    // A caller that took getDataPtr() before the tensor was computed keeps reading
    // through that pointer afterwards (the reference's tests do: there the pointer
    // is the data). If a host mirror of the right size exists, bring it up to date
    // in place; Operator::compute() calls this for its outputs.
    void refreshHostMirrorInPlace();
    // Counts the writes to this tensor's values (dataRand, setData, a kernel's
    // output, a host pointer handed out): lets a holder of derived data, such as
    // repacked filters, see that it is out of date.
    uint64_t dataVersion() const { return version; }
    // Marks every tensor computed (directly or not) from this one as not
    // computed; dataRand and setData call it.
    void invalidateDependents();

    size_t getOffset(const Dim &pos) const; // (size_t)-1 when out of range

    // Row-major position cursor over the tensor's index space, as the
    // reference's tests walk outputs (include/tensor.h:275-304).
    void itInit() { it.assign(dims.size(), 0); }
    void itReset() { itInit(); }
    bool itValid() const;
    const Dim &itGet() const { return it; }
    void itNext();

    // splitting points (kept for the search-side API)
    const SplittingPoints *getSplittingPoints() const { return &splittingPoints; }
    bool setSplittingPoints(SplittingPoints v) {
        splittingPoints = std::move(v);
        return true;
    }
    void initSplittingPoints() { splittingPoints.assign(dims.size(), {}); }

    void print();
    void printShape();

  private:
    const size_t guid;
    uint64_t hash;
    Dim dims;
    OpVec inputOf;
    Operator *outputOf = nullptr;
    DataType dtype;
    TensorType type;
    ComputeState computed = NotComputed;
    SplittingPoints splittingPoints;
    Dim dimPenalty;
    Dim it;

    float *dev = nullptr;
    size_t devElems = 0;
    bool ownsDev = false;
    std::vector<VType> host;
    bool hostFresh = false; // host mirror holds the current values
    bool devFresh = false;  // device buffer holds the current values
    uint64_t version = 0;
};

void printTensor(Tensor *tensor);

} // namespace tpm
