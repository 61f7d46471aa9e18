// Core types of the operator layer: error codes, tensor views, and the per-caller context that owns
// scratch memory.  The public interface is the one MatConvNet's operator library exposes
// (matlab/src/bits/data.hpp:38-266) so that code written against vl::Tensor / vl::Context keeps
// compiling; the GPU device type is backed by HIP on gfx950 instead of CUDA.
#ifndef MCN_AMD_BITS_DATA_HPP
#define MCN_AMD_BITS_DATA_HPP

#include <cstddef>
#include <string>

#define VL_TENSOR_SHAPE_MAX_NUM_DIMENSIONS 8

namespace vl {

// Values are part of the contract (bits/data.hpp:38-52): the C ABI returns the same numbers.
enum ErrorCode {
  VLE_Success = 0,
  VLE_Unsupported,
  VLE_Cuda,  // device runtime error; kept under its historical name, raised for HIP errors here
  VLE_Cudnn,
  VLE_Cublas,
  VLE_OutOfMemory,
  VLE_OutOfGPUMemeory,
  VLE_IllegalArgument,
  VLE_Unknown,
  VLE_Timeout,
  VLE_NoData,
  VLE_IllegalMessage,
  VLE_Interrupted
};

// Generic description of a code.  Unlike bits/data.cu:83-96 every enumerator has its own entry.
const char* getErrorMessage(ErrorCode error);

enum DeviceType { VLDT_CPU = 0, VLDT_GPU };
enum DataType { VLDT_Char, VLDT_Float, VLDT_Double };

template <DataType id> struct DataTypeTraits {};
template <> struct DataTypeTraits<VLDT_Char> { typedef char type; static constexpr std::size_t size = sizeof(char); };
template <> struct DataTypeTraits<VLDT_Float> { typedef float type; static constexpr std::size_t size = sizeof(float); };
template <> struct DataTypeTraits<VLDT_Double> { typedef double type; static constexpr std::size_t size = sizeof(double); };

template <typename type> struct BuiltinToDataType {};
template <> struct BuiltinToDataType<char> { enum { dataType = VLDT_Char }; };
template <> struct BuiltinToDataType<float> { enum { dataType = VLDT_Float }; };
template <> struct BuiltinToDataType<double> { enum { dataType = VLDT_Double }; };

inline std::size_t getDataTypeSizeInBytes(DataType dataType) {
  return dataType == VLDT_Char ? 1 : dataType == VLDT_Float ? 4 : dataType == VLDT_Double ? 8 : 0;
}

inline int divideAndRoundUp(int a, int b) { return (a + b - 1) / b; }
inline std::size_t divideAndRoundUp(std::size_t a, std::size_t b) { return (a + b - 1) / b; }

// g = gcd(a,b) together with Bezout coefficients a*u + b*v = g.
int gcd(int a, int b, int& u, int& v);
// Standard normal deviate (Box-Muller on rand()).
double randn();
// Monotonic clock in microseconds.
std::size_t getTime();

class HipHelper;  // stream + HIP error capture; the role CudaHelper plays in bits/datacu.hpp

namespace impl {
// Grow-only block of memory on one device: reallocated only when a larger size or another type is asked.
class Buffer {
 public:
  Buffer();
  ErrorCode init(DeviceType deviceType, DataType dataType, std::size_t size);
  void* getMemory();
  int getNumReallocations() const;
  void clear();
  void invalidateGpu();  // forget a device allocation without freeing it (after a device reset)

 protected:
  DeviceType deviceType;
  DataType dataType;
  std::size_t size;
  void* memory;
  int numReallocations;
};
}  // namespace impl

// Scratch memory, the all-ones vector, the stream and the last error of one caller.  Not thread safe,
// like the reference's (one static context per MEX file, used from MATLAB's single thread).
class Context {
 public:
  Context();
  ~Context();

  void* getWorkspace(DeviceType device, std::size_t size);
  void clearWorkspace(DeviceType device);
  void* getAllOnes(DeviceType device, DataType type, std::size_t size);
  void clearAllOnes(DeviceType device);
  HipHelper& getHipHelper();

  void clear();          // release everything
  void invalidateGpu();  // drop device memory and handles without touching the device

  ErrorCode passError(ErrorCode error, char const* message = NULL);
  ErrorCode setError(ErrorCode error, char const* message = NULL);
  void resetLastError();
  ErrorCode getLastError() const;
  std::string const& getLastErrorMessage() const;

 private:
  Context(Context const&);
  Context& operator=(Context const&);
  impl::Buffer workspace[2];
  impl::Buffer allOnes[2];
  ErrorCode lastError;
  std::string lastErrorMessage;
  HipHelper* hipHelper;
};

// Up to 8 extents; extents past the rank read as 1; rank 0 means "empty".
class TensorShape {
 public:
  TensorShape();
  TensorShape(TensorShape const& t);
  TensorShape(std::size_t height, std::size_t width, std::size_t depth, std::size_t size);
  TensorShape(std::size_t const* dimensions, std::size_t numDimensions);

  void clear();
  void setDimension(std::size_t num, std::size_t dimension);
  void setDimensions(std::size_t const* dimensions, std::size_t numDimensions);
  void setHeight(std::size_t x);
  void setWidth(std::size_t x);
  void setDepth(std::size_t x);
  void setSize(std::size_t x);
  void reshape(std::size_t numDimensions);  // fold trailing extents into the last kept one, or pad with 1
  void reshape(TensorShape const& shape);

  std::size_t getDimension(std::size_t num) const;
  std::size_t const* getDimensions() const;
  std::size_t getNumDimensions() const;
  std::size_t getHeight() const;
  std::size_t getWidth() const;
  std::size_t getDepth() const;
  std::size_t getSize() const;
  std::size_t getNumElements() const;
  bool isEmpty() const;

 protected:
  std::size_t dimensions[VL_TENSOR_SHAPE_MAX_NUM_DIMENSIONS];
  std::size_t numDimensions;
};

bool operator==(TensorShape const& a, TensorShape const& b);
inline bool operator!=(TensorShape const& a, TensorShape const& b) { return !(a == b); }

// Non-owning view: shape + element type + device + pointer.  A null pointer means "argument absent".
class Tensor : public TensorShape {
 public:
  Tensor();
  Tensor(Tensor const&);
  Tensor(TensorShape const& shape, DataType dataType, DeviceType deviceType, void* memory, std::size_t memorySize);
  void* getMemory();
  void const* getMemory() const;
  DeviceType getDeviceType() const;
  TensorShape getShape() const;
  DataType getDataType() const;
  operator bool() const;
  bool isNull() const;
  void setMemory(void* x);

 protected:
  DeviceType deviceType;
  DataType dataType;
  void* memory;
  std::size_t memorySize;
};

inline bool areCompatible(Tensor const& a, Tensor const& b) {
  if (a.isEmpty() || a.isNull() || b.isEmpty() || b.isNull()) return true;
  return a.getDeviceType() == b.getDeviceType() && a.getDataType() == b.getDataType();
}

}  // namespace vl
#endif
