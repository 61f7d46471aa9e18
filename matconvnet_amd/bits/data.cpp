// Implementation of the core types declared in data.hpp.
#include "data.hpp"

#include <cassert>
#include <chrono>
#include <cmath>
#include <cstdlib>
#include <cstring>

#include <hip/hip_runtime_api.h>

#include "../../include/mcn_hip.h"
#include "hiphelper.hpp"

namespace vl {

const char* getErrorMessage(ErrorCode error) {
  switch (error) {
    case VLE_Success: return "success";
    case VLE_Unsupported: return "unsupported feature error";
    case VLE_Cuda: return "HIP error";
    case VLE_Cudnn: return "cuDNN error";
    case VLE_Cublas: return "cuBLAS error";
    case VLE_OutOfMemory: return "out of memory error";
    case VLE_OutOfGPUMemeory: return "out of GPU memory error";
    case VLE_IllegalArgument: return "illegal argument error";
    case VLE_Timeout: return "timeout";
    case VLE_NoData: return "no data";
    case VLE_IllegalMessage: return "illegal message";
    case VLE_Interrupted: return "interrupted";
    default: return "unknown error";
  }
}

int gcd(int a, int b, int& u, int& v) {
  // extended Euclid, iterative
  int u0 = 1, v0 = 0, u1 = 0, v1 = 1;
  while (b != 0) {
    const int q = a / b;
    int t = a - q * b; a = b; b = t;
    t = u0 - q * u1; u0 = u1; u1 = t;
    t = v0 - q * v1; v0 = v1; v1 = t;
  }
  u = u0;
  v = v0;
  return a;
}

double randn() {
  const double twoPi = 6.283185307179586476925286766559;
  double u1;
  do { u1 = (std::rand() + 1.0) / (RAND_MAX + 2.0); } while (u1 <= 0.0);
  const double u2 = (std::rand() + 1.0) / (RAND_MAX + 2.0);
  return std::sqrt(-2.0 * std::log(u1)) * std::cos(twoPi * u2);
}

std::size_t getTime() {
  using namespace std::chrono;
  return (std::size_t)duration_cast<microseconds>(steady_clock::now().time_since_epoch()).count();
}

// --------------------------------------------------------------------------------------------- Buffer

namespace impl {

Buffer::Buffer() : deviceType(VLDT_CPU), dataType(VLDT_Char), size(0), memory(NULL), numReallocations(0) {}

void* Buffer::getMemory() { return memory; }
int Buffer::getNumReallocations() const { return numReallocations; }

ErrorCode Buffer::init(DeviceType wantDevice, DataType wantType, std::size_t wantSize) {
  if (memory != NULL && deviceType == wantDevice && dataType == wantType && size >= wantSize) return VLE_Success;
  clear();
  const std::size_t bytes = getDataTypeSizeInBytes(wantType) * wantSize;
  void* fresh = NULL;
  if (wantDevice == VLDT_CPU) {
    fresh = std::malloc(bytes ? bytes : 1);
    if (fresh == NULL) return VLE_OutOfMemory;
  } else {
    if (hipMalloc(&fresh, bytes ? bytes : 1) != hipSuccess) {
      (void)hipGetLastError();
      return VLE_OutOfMemory;  // the reference reports device exhaustion with the same code (data.cu:216)
    }
  }
  deviceType = wantDevice;
  dataType = wantType;
  size = wantSize;
  memory = fresh;
  ++numReallocations;
  return VLE_Success;
}

void Buffer::clear() {
  if (memory != NULL) {
    if (deviceType == VLDT_CPU) std::free(memory);
    else (void)hipFree(memory);
  }
  memory = NULL;
  size = 0;
}

void Buffer::invalidateGpu() {
  if (deviceType == VLDT_GPU) {
    memory = NULL;
    size = 0;
  }
}

}  // namespace impl

// ------------------------------------------------------------------------------------------ HipHelper

HipHelper::HipHelper() : stream(NULL) {}
void* HipHelper::getStream() const { return stream; }
ErrorCode HipHelper::setStream(void* s) { stream = s; return VLE_Success; }
std::string const& HipHelper::getLastHipErrorMessage() const { return lastMessage; }
void HipHelper::clear() { stream = NULL; lastMessage.clear(); }
void HipHelper::invalidateGpu() { stream = NULL; }

ErrorCode HipHelper::catchHipError(char const* description) {
  hipError_t e = hipPeekAtLastError();
  if (e == hipSuccess) return VLE_Success;
  (void)hipGetLastError();
  lastMessage = std::string(description ? description : "HIP") + ": " + hipGetErrorString(e);
  return VLE_Cuda;
}

// -------------------------------------------------------------------------------------------- Context

Context::Context() : lastError(VLE_Success), hipHelper(NULL) {}
Context::~Context() { clear(); }

void Context::clear() {
  for (int d = 0; d < 2; ++d) {
    workspace[d].clear();
    allOnes[d].clear();
  }
  if (hipHelper) {
    delete hipHelper;
    hipHelper = NULL;
  }
  resetLastError();
}

void Context::invalidateGpu() {
  workspace[VLDT_GPU].invalidateGpu();
  allOnes[VLDT_GPU].invalidateGpu();
  if (hipHelper) hipHelper->invalidateGpu();
}

HipHelper& Context::getHipHelper() {
  if (!hipHelper) hipHelper = new HipHelper();
  return *hipHelper;
}

void* Context::getWorkspace(DeviceType device, std::size_t bytes) {
  ErrorCode e = workspace[device].init(device, VLDT_Char, bytes);
  if (e != VLE_Success) {
    setError(e, "getWorkspace");
    return NULL;
  }
  return workspace[device].getMemory();
}

void Context::clearWorkspace(DeviceType device) { workspace[device].clear(); }

void* Context::getAllOnes(DeviceType device, DataType type, std::size_t count) {
  const int before = allOnes[device].getNumReallocations();
  ErrorCode e = allOnes[device].init(device, type, count);
  void* data = NULL;
  if (e == VLE_Success) {
    data = allOnes[device].getMemory();
    if (allOnes[device].getNumReallocations() > before) {  // new block: fill it
      if (device == VLDT_CPU) {
        if (type == VLDT_Float) for (std::size_t i = 0; i < count; ++i) ((float*)data)[i] = 1.0f;
        else if (type == VLDT_Double) for (std::size_t i = 0; i < count; ++i) ((double*)data)[i] = 1.0;
        else std::memset(data, 1, count);
      } else if (type == VLDT_Float) {
        if (mcn_fill(getHipHelper().getStream(), (float*)data, 1.0f, count) != MCN_SUCCESS) e = VLE_Cuda;
      } else {
        e = VLE_Unsupported;  // only single precision exists on the HIP device
      }
    }
  }
  if (setError(e, "getAllOnes: ") != VLE_Success) return NULL;
  return data;
}

void Context::clearAllOnes(DeviceType device) { allOnes[device].clear(); }

void Context::resetLastError() {
  lastError = VLE_Success;
  lastErrorMessage.clear();
}

ErrorCode Context::passError(ErrorCode error, char const* description) {
  if (error != VLE_Success && description) lastErrorMessage = std::string(description) + ": " + lastErrorMessage;
  return error;
}

ErrorCode Context::setError(ErrorCode error, char const* description) {
  if (error == VLE_Success) return error;
  lastError = error;
  std::string text = getErrorMessage(error);
  if (description) text = std::string(description) + " [" + text + "]";
  if (error == VLE_Cuda && hipHelper && !hipHelper->getLastHipErrorMessage().empty())
    text += " [hip: " + hipHelper->getLastHipErrorMessage() + "]";
  lastErrorMessage = text;
  return error;
}

ErrorCode Context::getLastError() const { return lastError; }
std::string const& Context::getLastErrorMessage() const { return lastErrorMessage; }

// ---------------------------------------------------------------------------------------- TensorShape

TensorShape::TensorShape() : numDimensions(0) {}
TensorShape::TensorShape(TensorShape const& t) : numDimensions(t.numDimensions) {
  for (std::size_t k = 0; k < numDimensions; ++k) dimensions[k] = t.dimensions[k];
}
TensorShape::TensorShape(std::size_t h, std::size_t w, std::size_t d, std::size_t n) : numDimensions(4) {
  dimensions[0] = h; dimensions[1] = w; dimensions[2] = d; dimensions[3] = n;
}
TensorShape::TensorShape(std::size_t const* dims, std::size_t count) : numDimensions(0) { setDimensions(dims, count); }

void TensorShape::clear() { numDimensions = 0; }

void TensorShape::setDimensions(std::size_t const* dims, std::size_t count) {
  assert(count <= VL_TENSOR_SHAPE_MAX_NUM_DIMENSIONS);
  for (std::size_t k = 0; k < count; ++k) dimensions[k] = dims[k];
  numDimensions = count;
}

void TensorShape::setDimension(std::size_t num, std::size_t dimension) {
  assert(num < VL_TENSOR_SHAPE_MAX_NUM_DIMENSIONS);
  if (num >= numDimensions) {
    // extents created on the way are 1 for a non-empty shape and 0 for an empty one
    const std::size_t filler = getNumElements() > 0 ? 1 : 0;
    for (std::size_t k = numDimensions; k < num; ++k) dimensions[k] = filler;
    numDimensions = num + 1;
  }
  dimensions[num] = dimension;
}

std::size_t TensorShape::getDimension(std::size_t num) const { return num < numDimensions ? dimensions[num] : 1; }
std::size_t const* TensorShape::getDimensions() const { return dimensions; }
std::size_t TensorShape::getNumDimensions() const { return numDimensions; }

std::size_t TensorShape::getNumElements() const {
  if (numDimensions == 0) return 0;
  std::size_t n = 1;
  for (std::size_t k = 0; k < numDimensions; ++k) n *= dimensions[k];
  return n;
}

std::size_t TensorShape::getHeight() const { return getDimension(0); }
std::size_t TensorShape::getWidth() const { return getDimension(1); }
std::size_t TensorShape::getDepth() const { return getDimension(2); }
std::size_t TensorShape::getSize() const { return getDimension(3); }
void TensorShape::setHeight(std::size_t x) { setDimension(0, x); }
void TensorShape::setWidth(std::size_t x) { setDimension(1, x); }
void TensorShape::setDepth(std::size_t x) { setDimension(2, x); }
void TensorShape::setSize(std::size_t x) { setDimension(3, x); }
bool TensorShape::isEmpty() const { return getNumElements() == 0; }

void TensorShape::reshape(std::size_t count) {
  assert(count <= VL_TENSOR_SHAPE_MAX_NUM_DIMENSIONS);
  const std::size_t total = getNumElements();
  if (count == 0) {
    numDimensions = 0;
    return;
  }
  setDimension(count - 1, 1);  // stretches if needed; the last kept extent is recomputed below
  numDimensions = count;
  const std::size_t kept = getNumElements();
  if (kept != 0) dimensions[count - 1] *= total / kept;
  else if (total == 0) dimensions[count - 1] = 0;
}

void TensorShape::reshape(TensorShape const& shape) { *this = shape; }

bool operator==(TensorShape const& a, TensorShape const& b) {
  if (a.getNumDimensions() != b.getNumDimensions()) return false;
  for (std::size_t k = 0; k < a.getNumDimensions(); ++k)
    if (a.getDimensions()[k] != b.getDimensions()[k]) return false;
  return true;
}

// --------------------------------------------------------------------------------------------- Tensor

Tensor::Tensor() : TensorShape(), deviceType(VLDT_CPU), dataType(VLDT_Float), memory(NULL), memorySize(0) {}
Tensor::Tensor(Tensor const& t)
    : TensorShape(t), deviceType(t.deviceType), dataType(t.dataType), memory(t.memory), memorySize(t.memorySize) {}
Tensor::Tensor(TensorShape const& shape, DataType dt, DeviceType dev, void* mem, std::size_t bytes)
    : TensorShape(shape), deviceType(dev), dataType(dt), memory(mem), memorySize(bytes) {}
void* Tensor::getMemory() { return memory; }
void const* Tensor::getMemory() const { return memory; }
DeviceType Tensor::getDeviceType() const { return deviceType; }
TensorShape Tensor::getShape() const { return TensorShape(*this); }
DataType Tensor::getDataType() const { return dataType; }
Tensor::operator bool() const { return memory != NULL; }
bool Tensor::isNull() const { return memory == NULL; }
void Tensor::setMemory(void* x) { memory = x; }

}  // namespace vl
