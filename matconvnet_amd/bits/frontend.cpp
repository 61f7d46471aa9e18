// See frontend.hpp.  Error texts are the reference drivers' own, so callers that match on them keep working.
#include "frontend.hpp"

#include "accumulate.hpp"

#include <cctype>
#include <cstdio>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "../../include/mcn_hip.h"
#include "hiphelper.hpp"

#include "nnbnorm.hpp"
#include "nnconv.hpp"
#include "nnpooling.hpp"
#include "nnsubsample.hpp"

namespace vl { namespace frontend {

Arg Arg::array(Tensor const& t) {
  Arg a;
  a.kind = Array;
  a.tensor = t;
  return a;
}

Arg Arg::string(std::string const& s) {
  Arg a;
  a.kind = String;
  a.text = s;
  return a;
}

Arg Arg::numeric(std::vector<double> const& values) {
  Arg a;
  a.kind = Array;
  a.owned.reset(new std::vector<double>(values));
  std::size_t dims[2] = {values.empty() ? 0u : 1u, values.size()};
  a.tensor = Tensor(TensorShape(dims, 2), VLDT_Double, VLDT_CPU, values.empty() ? NULL : &(*a.owned)[0],
                    values.size() * sizeof(double));
  return a;
}

namespace {

struct Failure {
  ErrorCode code;
  std::string text;
};

[[noreturn]] void raise(ErrorCode code, std::string const& text) {
  Failure f = {code, text};
  throw f;
}

bool sameTextNoCase(std::string const& a, char const* b) {
  std::size_t i = 0;
  for (; i < a.size() && b[i]; ++i)
    if (std::tolower((unsigned char)a[i]) != std::tolower((unsigned char)b[i])) return false;
  return i == a.size() && b[i] == 0;
}

struct OptionSpec {
  char const* name;
  bool hasArgument;
  int code;
};

// Walks "name, value, name, ..." like vlmxNextOption (matlab/src/bits/mexutils.h:470-562): names are
// matched without regard to case; unknown names and missing values are errors.
int nextOption(Arg const* in, int nin, OptionSpec const* specs, int* next, Arg const** value) {
  if (*next >= nin) return -1;
  Arg const& nameArg = in[*next];
  char buffer[160];
  if (nameArg.kind != Arg::String) {
    std::snprintf(buffer, sizeof(buffer), "The option name is not a string (argument number %d)", *next + 1);
    raise(VLE_IllegalArgument, buffer);
  }
  ++*next;
  for (int i = 0; specs[i].name; ++i) {
    if (!sameTextNoCase(nameArg.text, specs[i].name)) continue;
    if (!specs[i].hasArgument) {
      *value = NULL;
      return specs[i].code;
    }
    if (*next >= nin) {
      std::snprintf(buffer, sizeof(buffer), "Option '%s' requires an argument.", specs[i].name);
      raise(VLE_IllegalArgument, buffer);
    }
    *value = &in[*next];
    ++*next;
    return specs[i].code;
  }
  raise(VLE_IllegalArgument, "Unknown option '" + nameArg.text + "'.");
}

// "plain matrix": a real, full, double host array (vlmxIsPlainMatrix).
bool isPlainMatrix(Arg const& a) {
  return a.kind == Arg::Array && a.tensor.getDeviceType() == VLDT_CPU && a.tensor.getDataType() == VLDT_Double &&
         a.tensor.getNumDimensions() <= 2 && (a.tensor.getNumElements() == 0 || !a.tensor.isNull());
}

double const* values(Arg const& a) { return (double const*)a.tensor.getMemory(); }

void readPair(Arg const& a, char const* NAME, int* y, int* x) {
  if (!isPlainMatrix(a)) raise(VLE_IllegalArgument, std::string(NAME) + " is not a plain matrix.");
  switch (a.tensor.getNumElements()) {
    case 1: *y = *x = (int)values(a)[0]; break;
    case 2: *y = (int)values(a)[0]; *x = (int)values(a)[1]; break;
    default: raise(VLE_IllegalArgument, std::string(NAME) + " has neither one nor two elements.");
  }
}

void readPad(Arg const& a, int* top, int* bottom, int* left, int* right) {
  if (!isPlainMatrix(a)) raise(VLE_IllegalArgument, "PAD is not a plain matrix.");
  switch (a.tensor.getNumElements()) {
    case 1: *top = *bottom = *left = *right = (int)values(a)[0]; break;
    case 4:
      *top = (int)values(a)[0]; *bottom = (int)values(a)[1]; *left = (int)values(a)[2]; *right = (int)values(a)[3];
      break;
    default: raise(VLE_IllegalArgument, "PAD has neither one nor four elements.");
  }
}

// Data arguments: numeric arrays of class single or double (MexTensor::init, bits/datamex.cu:339-434).
Tensor dataTensor(Arg const& a, char const* NAME, std::size_t rank) {
  if (a.kind != Arg::Array) raise(VLE_IllegalArgument, std::string(NAME) + " is not a numeric array.");
  if (a.tensor.getDataType() != VLDT_Float && a.tensor.getDataType() != VLDT_Double)
    raise(VLE_IllegalArgument, std::string(NAME) + " is neither SINGLE nor DOUBLE.");
  Tensor t(a.tensor);
  t.reshape(rank);
  return t;
}

Tensor emptyMatrix(DataType type) {
  std::size_t dims[2] = {0, 0};
  return Tensor(TensorShape(dims, 2), type, VLDT_CPU, NULL, 0);
}

// Uninitialised output of a given shape on the device/type of the data (MexTensor::init with a shape).
Tensor newOutput(Allocator& allocator, DeviceType device, DataType type, TensorShape const& shape) {
  const std::size_t bytes = shape.getNumElements() * getDataTypeSizeInBytes(type);
  void* memory = NULL;
  if (bytes > 0) {
    memory = allocator.allocate(device, bytes);
    if (!memory) raise(device == VLDT_GPU ? VLE_OutOfGPUMemeory : VLE_OutOfMemory, "Could not allocate an output array.");
  }
  return Tensor(shape, type, device, memory, bytes);
}

void failFromContext(Context& context, ErrorCode e) {
  if (e != VLE_Success) raise(e, context.getLastErrorMessage());
}

// ------------------------------------------------------------------------------------------ vl_nnconv

void nnconv(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in) {
  enum { optStride, optPad, optDilate, optVerbose, optNoDerData, optNoDerFilters, optNoDerBiases, optCudnn, optNoCudnn, optCudnnWs };
  static OptionSpec const specs[] = {
      {"Stride", true, optStride}, {"Pad", true, optPad}, {"Dilate", true, optDilate}, {"Verbose", false, optVerbose},
      {"NoDerData", false, optNoDerData}, {"NoDerFilters", false, optNoDerFilters}, {"NoderBiases", false, optNoDerBiases},
      {"Cudnn", false, optCudnn}, {"NoCudnn", false, optNoCudnn}, {"CudnnWorkSpaceLimit", true, optCudnnWs}, {NULL, false, 0}};
  int strideX = 1, strideY = 1, padLeft = 0, padRight = 0, padTop = 0, padBottom = 0, dilateX = 1, dilateY = 1;
  bool wantDerData = true, wantDerFilters = true, wantDerBiases = true;

  if (nin < 3) raise(VLE_IllegalArgument, "There are less than three arguments.");
  int next = 4;
  bool backMode;
  if (nin > 3 && in[3].kind == Arg::String) {
    next = 3;
    backMode = false;
  } else {
    backMode = nin >= 4;
  }
  int opt;
  Arg const* value = NULL;
  while ((opt = nextOption(in, nin, specs, &next, &value)) >= 0) {
    switch (opt) {
      case optStride: readPair(*value, "STRIDE", &strideY, &strideX); break;
      case optPad: readPad(*value, &padTop, &padBottom, &padLeft, &padRight); break;
      case optDilate: readPair(*value, "DILATE", &dilateY, &dilateX); break;
      case optNoDerData: wantDerData = false; break;
      case optNoDerFilters: wantDerFilters = false; break;
      case optNoDerBiases: wantDerBiases = false; break;
      default: break;  // Verbose and the cuDNN switches have nothing to act on here
    }
  }

  Tensor data = dataTensor(in[0], "DATA", 4);
  Tensor filters = dataTensor(in[1], "FILTERS", 4);
  Tensor biases = dataTensor(in[2], "BIASES", in[2].tensor.getNumDimensions());
  Tensor derOutput;
  if (backMode) derOutput = dataTensor(in[3], "DEROUTPUT", 4);
  const bool hasFilters = !filters.isEmpty(), hasBiases = !biases.isEmpty();

  if (hasFilters && !areCompatible(data, filters)) raise(VLE_IllegalArgument, "DATA and FILTERS do not have compatible formats.");
  if (hasBiases && !areCompatible(data, biases)) raise(VLE_IllegalArgument, "DATA and BIASES do not have compatible formats.");
  if (backMode && !areCompatible(data, derOutput)) raise(VLE_IllegalArgument, "DATA and DEROUTPUT do not have compatible formats.");
  if (strideX < 1 || strideY < 1) raise(VLE_IllegalArgument, "At least one element of STRIDE is smaller than one.");
  if (padLeft < 0 || padRight < 0 || padTop < 0 || padBottom < 0) raise(VLE_IllegalArgument, "An element of PAD is negative.");
  if (dilateY < 1 || dilateX < 1) raise(VLE_IllegalArgument, "An element of DILATE is less than one.");
  if (!hasFilters && (dilateY != 1 || dilateX != 1)) raise(VLE_IllegalArgument, "There are no filters and DILATE is not one.");
  // the filter shape; empty FILTERS stand for the identity filter bank (vl_nnconv.cu:296-321)
  TensorShape filtersShape(filters);
  std::size_t equivalentNumFilters;
  if (hasFilters) {
    if (filtersShape.getHeight() == 0 || filtersShape.getWidth() == 0 || filtersShape.getDepth() == 0)
      raise(VLE_IllegalArgument, "A dimension of FILTERS is void.");
    if ((long)data.getHeight() + (padTop + padBottom) < ((long)filters.getHeight() - 1) * dilateY + 1 ||
        (long)data.getWidth() + (padLeft + padRight) < ((long)filters.getWidth() - 1) * dilateX + 1)
      raise(VLE_IllegalArgument, "FILTERS are larger than the DATA (including padding).");
    const std::size_t groups = data.getDepth() / filters.getDepth();
    if (groups * filters.getDepth() != data.getDepth()) raise(VLE_IllegalArgument, "The FILTERS depth does not divide the DATA depth.");
    if (groups == 0 || filters.getSize() % groups != 0)
      raise(VLE_IllegalArgument, "The number of filter groups does not divide the number of filters.");
    equivalentNumFilters = filters.getSize();
  } else {
    filtersShape = TensorShape(1, 1, data.getDepth(), data.getDepth());
    equivalentNumFilters = data.getDepth();
  }
  const long extentY = ((long)filtersShape.getHeight() - 1) * dilateY + 1, extentX = ((long)filtersShape.getWidth() - 1) * dilateX + 1;

  TensorShape outputShape(((long)data.getHeight() + (padTop + padBottom) - extentY) / strideY + 1,
                          ((long)data.getWidth() + (padLeft + padRight) - extentX) / strideX + 1, equivalentNumFilters,
                          data.getSize());
  if (backMode && (TensorShape(derOutput) != outputShape))
    raise(VLE_IllegalArgument, "DEROUTPUT dimensions are incompatible with X and FILTERS.");
  if (hasBiases && biases.getNumElements() != filtersShape.getSize())
    raise(VLE_IllegalArgument, "The number of elements of BIASES is not the same as the number of filters.");

  const DeviceType device = data.getDeviceType();
  const DataType type = data.getDataType();
  // (the reference's fully-connected special case, vl_nnconv.cu:343-358,424-433, is the same product: the general
  // kernels below cover 1 x 1 outputs)
  nn::Convolution op(context, strideY, strideX, padTop, padBottom, padLeft, padRight, dilateY, dilateX);
  nn::Subsample sub(context, strideY, strideX, padTop, padBottom, padLeft, padRight);  // no filters: subsample + bias
  Tensor noBias;
  if (!backMode) {
    Tensor output = newOutput(allocator, device, type, outputShape);
    failFromContext(context, hasFilters ? op.forward(output, 0, data, 1, filters, hasBiases ? biases : noBias)
                                        : sub.forwardWithBias(output, data, hasBiases ? biases : noBias));
    out[0] = output;
    return;
  }
  Tensor derData, derFilters, derBiases;
  if (wantDerData) derData = newOutput(allocator, device, type, data.getShape());
  if (wantDerFilters && hasFilters) derFilters = newOutput(allocator, device, type, filters.getShape());
  if (wantDerBiases && hasBiases) derBiases = newOutput(allocator, device, type, biases.getShape());
  failFromContext(context, hasFilters ? op.backward(derData, derFilters, derBiases, data, filters, derOutput)
                                      : sub.backwardWithBias(derData, derBiases, derOutput));
  const DataType outType = derOutput.getDataType();
  out[0] = wantDerData ? derData : emptyMatrix(outType);
  if (nout > 1) out[1] = (wantDerFilters && hasFilters) ? derFilters : emptyMatrix(outType);
  if (nout > 2) out[2] = (wantDerBiases && hasBiases) ? derBiases : emptyMatrix(outType);
}

// ----------------------------------------------------------------------------------------- vl_nnconvt

void nnconvt(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in) {
  enum { optUpsample, optCrop, optVerbose, optNumGroups, optNoDerData, optNoDerFilters, optNoDerBiases, optCudnn, optNoCudnn, optCudnnWs };
  static OptionSpec const specs[] = {
      {"Upsample", true, optUpsample}, {"Crop", true, optCrop}, {"Verbose", false, optVerbose}, {"NumGroups", true, optNumGroups},
      {"NoDerData", false, optNoDerData}, {"NoDerFilters", false, optNoDerFilters}, {"NoDerBiases", false, optNoDerBiases},
      {"CUDNN", false, optCudnn}, {"NoCUDNN", false, optNoCudnn}, {"CudnnWorkSpaceLimit", true, optCudnnWs}, {NULL, false, 0}};
  int upsampleX = 1, upsampleY = 1, cropLeft = 0, cropRight = 0, cropTop = 0, cropBottom = 0, numFilterGroups = 1;
  bool wantDerData = true, wantDerFilters = true, wantDerBiases = true;

  if (nin < 3) raise(VLE_IllegalArgument, "There are less than three arguments.");
  int next = 4;
  bool backMode;
  if (nin > 3 && in[3].kind == Arg::String) {
    next = 3;
    backMode = false;
  } else {
    backMode = nin >= 4;
  }
  int opt;
  Arg const* value = NULL;
  while ((opt = nextOption(in, nin, specs, &next, &value)) >= 0) {
    switch (opt) {
      case optUpsample:  // texts as in vl_nnconvt.cu:128-142
        if (!isPlainMatrix(*value)) raise(VLE_IllegalArgument, "upsample is not a plain matrix.");
        switch (value->tensor.getNumElements()) {
          case 1: upsampleY = upsampleX = (int)values(*value)[0]; break;
          case 2: upsampleY = (int)values(*value)[0]; upsampleX = (int)values(*value)[1]; break;
          default: raise(VLE_IllegalArgument, "upsample has neither one nor two elements.");
        }
        break;
      case optCrop:  // vl_nnconvt.cu:145-164
        if (!isPlainMatrix(*value)) raise(VLE_IllegalArgument, "crop is not a plain matrix.");
        switch (value->tensor.getNumElements()) {
          case 1: cropLeft = cropRight = cropTop = cropBottom = (int)values(*value)[0]; break;
          case 4:
            cropTop = (int)values(*value)[0]; cropBottom = (int)values(*value)[1]; cropLeft = (int)values(*value)[2];
            cropRight = (int)values(*value)[3];
            break;
          default: raise(VLE_IllegalArgument, "crop has neither one nor two elements.");
        }
        break;
      case optNumGroups:
        if (!isPlainMatrix(*value) || value->tensor.getNumElements() != 1) raise(VLE_IllegalArgument, "NUMGROUPS is not a plain scalar.");
        numFilterGroups = (int)values(*value)[0];
        break;
      case optNoDerData: wantDerData = false; break;
      case optNoDerFilters: wantDerFilters = false; break;
      case optNoDerBiases: wantDerBiases = false; break;
      default: break;
    }
  }

  Tensor data = dataTensor(in[0], "DATA", 4);
  Tensor filters = dataTensor(in[1], "FILTERS", 4);
  Tensor biases = dataTensor(in[2], "BIASES", in[2].tensor.getNumDimensions());
  Tensor derOutput;
  if (backMode) derOutput = dataTensor(in[3], "DEROUTPUT", 4);
  const bool hasBiases = !biases.isEmpty();

  if (!areCompatible(data, filters)) raise(VLE_IllegalArgument, "DATA and FILTERS do not have compatible formats.");
  if (hasBiases && !areCompatible(data, biases)) raise(VLE_IllegalArgument, "DATA and BIASES do not have compatible formats.");
  if (backMode && !areCompatible(data, derOutput)) raise(VLE_IllegalArgument, "DATA and DEROUTPUT do not have compatible formats.");
  if (upsampleX < 1 || upsampleY < 1) raise(VLE_IllegalArgument, "At least one element of UPSAMPLE is smaller than one.");
  if (cropLeft < 0 || cropRight < 0 || cropTop < 0 || cropBottom < 0) raise(VLE_IllegalArgument, "An element of CROP is negative.");

  TensorShape filtersShape(filters);
  if (filtersShape.getHeight() == 0 || filtersShape.getWidth() == 0 || filtersShape.getDepth() == 0)
    raise(VLE_IllegalArgument, "A dimension of FILTERS is void.");
  if (numFilterGroups < 1) raise(VLE_IllegalArgument, "NUMGROUPS is less than 1.");
  if (filters.getSize() % numFilterGroups != 0)
    raise(VLE_IllegalArgument,
          "The number of filter groups does not divide the filter bank depth (fourth dimension of FILTERS).");
  if (filters.getSize() != data.getDepth())
    raise(VLE_IllegalArgument,
          "The filter bank depth (fourth dimension of FILTERS) is not the same as the data depth (third dimension of X).");

  const long outH = ((long)data.getHeight() - 1) * upsampleY - (cropTop + cropBottom) + (long)filtersShape.getHeight();
  const long outW = ((long)data.getWidth() - 1) * upsampleX - (cropLeft + cropRight) + (long)filtersShape.getWidth();
  if (outH < 1 || outW < 1) raise(VLE_IllegalArgument, "The output array is empty due to CROP being too large.");
  TensorShape outputShape(outH, outW, filtersShape.getDepth() * numFilterGroups, data.getSize());
  if (backMode && (TensorShape(derOutput) != outputShape))
    raise(VLE_IllegalArgument, "DEROUTPUT dimensions are incompatible with X and FILTERS.");
  if (hasBiases && biases.getNumElements() != outputShape.getDepth())
    raise(VLE_IllegalArgument, "The number of elements of BIASES is not the same as the dimenison of the filters.");

  const DeviceType device = data.getDeviceType();
  const DataType type = data.getDataType();
  nn::ConvolutionTranspose op(context, upsampleY, upsampleX, cropTop, cropBottom, cropLeft, cropRight);
  Tensor noBias;
  if (!backMode) {
    Tensor output = newOutput(allocator, device, type, outputShape);
    failFromContext(context, op.forward(output, data, filters, hasBiases ? biases : noBias));
    out[0] = output;
    return;
  }
  Tensor derData, derFilters, derBiases;
  if (wantDerData) derData = newOutput(allocator, device, type, data.getShape());
  if (wantDerFilters) derFilters = newOutput(allocator, device, type, filters.getShape());
  if (wantDerBiases && hasBiases) derBiases = newOutput(allocator, device, type, biases.getShape());
  failFromContext(context, op.backward(derData, derFilters, derBiases, data, filters, derOutput));
  const DataType outType = derOutput.getDataType();
  out[0] = wantDerData ? derData : emptyMatrix(outType);
  if (nout > 1) out[1] = wantDerFilters ? derFilters : emptyMatrix(outType);
  if (nout > 2) out[2] = (wantDerBiases && hasBiases) ? derBiases : emptyMatrix(outType);
}

// ----------------------------------------------------------------------------------------- vl_nnbnorm

void nnbnorm(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in) {
  enum { optVerbose, optEpsilon, optMoments, optCudnn, optNoCudnn };
  static OptionSpec const specs[] = {{"Verbose", false, optVerbose}, {"Epsilon", true, optEpsilon}, {"Moments", true, optMoments},
                                     {"Cudnn", false, optCudnn}, {"NoCudnn", false, optNoCudnn}, {NULL, false, 0}};
  double epsilon = 1e-4;
  if (nin < 3) raise(VLE_IllegalArgument, "The arguments are less than three.");
  int next = 4;
  bool backMode;
  if (nin > 3 && in[3].kind == Arg::String) {
    next = 3;
    backMode = false;
  } else {
    backMode = nin >= 4;
  }
  const bool returnMoments = backMode ? (nout > 3) : (nout > 1);
  Arg const* momentsArg = NULL;
  int opt;
  Arg const* value = NULL;
  while ((opt = nextOption(in, nin, specs, &next, &value)) >= 0) {
    switch (opt) {
      case optEpsilon:
        if (!isPlainMatrix(*value) || value->tensor.getNumElements() != 1) raise(VLE_IllegalArgument, "EPSILON is not a plain scalar.");
        epsilon = values(*value)[0];
        break;
      case optMoments: momentsArg = value; break;
      default: break;
    }
  }
  const bool givenMoments = momentsArg != NULL;

  Tensor data = dataTensor(in[0], "DATA", 4);
  Tensor multipliers = dataTensor(in[1], "MULTIPLIERS", 1);
  Tensor biases = dataTensor(in[2], "BIASES", 1);
  Tensor derOutput, moments;
  if (backMode) derOutput = dataTensor(in[3], "DEROUTPUT", 4);
  if (givenMoments) moments = dataTensor(*momentsArg, "MOMENTS", 2);

  if (!areCompatible(data, multipliers)) raise(VLE_IllegalArgument, "DATA and MULTIPLIERS do not have compatible formats.");
  if (!areCompatible(data, biases)) raise(VLE_IllegalArgument, "DATA and BIASES do not have compatible formats.");
  if (backMode && !areCompatible(data, derOutput)) raise(VLE_IllegalArgument, "DATA and DEROUTPUT do not have compatible formats.");
  if (backMode && (data.getShape() != derOutput.getShape())) raise(VLE_IllegalArgument, "DATA and DEROUTPUT do not have the same size.");
  if (givenMoments && !areCompatible(data, moments)) raise(VLE_IllegalArgument, "DATA and MOMENTS do not have compatible formats.");
  if (multipliers.getHeight() != data.getDepth()) raise(VLE_IllegalArgument, "The MULTIPLIERS size does not match the DATA depth.");
  if (biases.getHeight() != data.getDepth()) raise(VLE_IllegalArgument, "The BIASES size does not match the DATA depth.");
  if (givenMoments && moments.getNumElements() != 2 * data.getDepth())
    raise(VLE_IllegalArgument, "The MOMENTS size does not match the DATA depth.");

  const DeviceType device = data.getDeviceType();
  const DataType type = data.getDataType();
  if (returnMoments && !givenMoments) moments = newOutput(allocator, device, type, TensorShape(data.getDepth(), 2, 1, 1));

  nn::BatchNorm op(context, epsilon);
  if (!backMode) {
    Tensor output = newOutput(allocator, device, type, data.getShape());
    failFromContext(context, givenMoments ? op.forwardWithMoment(output, moments, data, multipliers, biases)
                                          : op.forward(output, moments, data, multipliers, biases));
    out[0] = output;
    if (nout > 1 && moments) out[1] = moments;
    return;
  }
  // derivatives of the parameters keep the shape the parameters were passed with
  Tensor derData = newOutput(allocator, device, type, data.getShape());
  Tensor derMultipliers = newOutput(allocator, device, type, in[1].tensor.getShape());
  Tensor derBiases = newOutput(allocator, device, type, in[2].tensor.getShape());
  failFromContext(context, givenMoments
                               ? op.backwardWithMoment(derData, derMultipliers, derBiases, moments, data, multipliers, biases, derOutput)
                               : op.backward(derData, derMultipliers, derBiases, moments, data, multipliers, biases, derOutput));
  out[0] = derData;
  if (nout > 1) out[1] = derMultipliers;
  if (nout > 2) out[2] = derBiases;
  if (nout > 3 && moments) out[3] = moments;
}

// ------------------------------------------------------------------------------------------ vl_nnpool

void nnpool(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in) {
  enum { optStride, optPad, optMethod, optVerbose, optCudnn, optNoCudnn };
  static OptionSpec const specs[] = {{"Stride", true, optStride}, {"Pad", true, optPad}, {"Method", true, optMethod},
                                     {"Verbose", false, optVerbose}, {"CUDNN", false, optCudnn}, {"NoCUDNN", false, optNoCudnn},
                                     {NULL, false, 0}};
  int poolWidth = 0, poolHeight = 0, strideX = 1, strideY = 1, padLeft = 0, padRight = 0, padTop = 0, padBottom = 0;
  nn::Pooling::Method method = nn::Pooling::Max;
  if (nin < 2) raise(VLE_IllegalArgument, "The arguments are less than two.");
  int next = 3;
  bool backMode;
  if (nin > 2 && in[2].kind == Arg::String) {
    next = 2;
    backMode = false;
  } else {
    backMode = nin >= 3;
  }
  int opt;
  Arg const* value = NULL;
  while ((opt = nextOption(in, nin, specs, &next, &value)) >= 0) {
    switch (opt) {
      case optStride: readPair(*value, "STRIDE", &strideY, &strideX); break;
      case optPad: readPad(*value, &padTop, &padBottom, &padLeft, &padRight); break;
      case optMethod:
        if (value->kind != Arg::String) raise(VLE_IllegalArgument, "METHOD is not a string.");
        if (sameTextNoCase(value->text, "max")) method = nn::Pooling::Max;
        else if (sameTextNoCase(value->text, "avg")) method = nn::Pooling::Average;
        else raise(VLE_IllegalArgument, "METHOD is not a supported method.");
        break;
      default: break;
    }
  }
  Tensor data = dataTensor(in[0], "DATA", 4);
  Tensor derOutput;
  if (backMode) derOutput = dataTensor(in[2], "DEROUTPUT", 4);
  if (backMode && !areCompatible(data, derOutput)) raise(VLE_IllegalArgument, "DATA and DEROUTPUT do not have compatible formats.");
  if (!isPlainMatrix(in[1])) raise(VLE_IllegalArgument, "SIZE is not a plain matrix.");
  switch (in[1].tensor.getNumElements()) {
    case 1: poolHeight = poolWidth = (int)values(in[1])[0]; break;
    case 2: poolHeight = (int)values(in[1])[0]; poolWidth = (int)values(in[1])[1]; break;
    default: raise(VLE_IllegalArgument, "SIZE has neither one nor two elements.");
  }
  if (strideX < 1 || strideY < 1) raise(VLE_IllegalArgument, "At least one element of STRIDE is smaller than one.");
  if (poolHeight == 0 || poolWidth == 0) raise(VLE_IllegalArgument, "A dimension of the pooling SIZE is void.");
  if ((long)data.getHeight() + (padTop + padBottom) < poolHeight || (long)data.getWidth() + (padLeft + padRight) < poolWidth)
    raise(VLE_IllegalArgument, "The pooling window is larger than the DATA (including padding).");
  if (padLeft < 0 || padRight < 0 || padTop < 0 || padBottom < 0) raise(VLE_IllegalArgument, "An element of PAD is negative.");
  if (padLeft >= poolWidth || padRight >= poolWidth || padTop >= poolHeight || padBottom >= poolHeight)
    raise(VLE_IllegalArgument, "A padding value is larger or equal to the size of the pooling window.");
  TensorShape outputShape(((long)data.getHeight() + (padTop + padBottom) - poolHeight) / strideY + 1,
                          ((long)data.getWidth() + (padLeft + padRight) - poolWidth) / strideX + 1, data.getDepth(),
                          data.getSize());
  if (backMode && (TensorShape(derOutput) != outputShape))
    raise(VLE_IllegalArgument, "DEROUTPUT dimensions are incompatible with X and POOL.");

  const DeviceType device = data.getDeviceType();
  const DataType type = data.getDataType();
  nn::Pooling op(context, poolHeight, poolWidth, strideY, strideX, padTop, padBottom, padLeft, padRight, method);
  if (!backMode) {
    Tensor output = newOutput(allocator, device, type, outputShape);
    failFromContext(context, op.forward(output, data));
    out[0] = output;
  } else {
    // The MEX driver zero-fills dzdx and lets the operator add into it (vl_nnpool.cu:255-259); the gather
    // kernel can write every element itself, which saves that pass over dzdx.
    Tensor derData = newOutput(allocator, device, type, data.getShape());
    failFromContext(context, op.backwardOverwrite(derData, data, derOutput));
    out[0] = derData;
  }
  (void)nout;
}

// ------------------------------------------------------------------------------------------ vl_taccum
// matlab/src/vl_taccummex.cu:151-224 (the MEX behind matlab/vl_taccum.m): (alpha, A, beta, B [, 'InPlace'])

void taccum(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in) {
  enum { optInPlace, optVerbose };
  static OptionSpec const specs[] = {{"InPlace", false, optInPlace}, {"Verbose", false, optVerbose}, {NULL, false, 0}};
  bool inplace = false;
  if (nin < 4) raise(VLE_IllegalArgument, "There are less than four arguments.");
  int next = 4, opt;
  Arg const* value = NULL;
  while ((opt = nextOption(in, nin, specs, &next, &value)) >= 0)
    if (opt == optInPlace) inplace = true;
  if (!(isPlainMatrix(in[0]) && in[0].tensor.getNumElements() == 1)) raise(VLE_IllegalArgument, "ALPHA is not a plain scalar.");
  if (!(isPlainMatrix(in[2]) && in[2].tensor.getNumElements() == 1)) raise(VLE_IllegalArgument, "BETA is not a plain scalar.");
  Tensor a = dataTensor(in[1], "A", 4), b = dataTensor(in[3], "B", 4);
  if (!areCompatible(a, b)) raise(VLE_IllegalArgument, "A and B do not have compatible formats.");
  if (a.getNumElements() != b.getNumElements()) raise(VLE_IllegalArgument, "A and B do not have the same number of elements.");
  const double alpha = values(in[0])[0], beta = values(in[2])[0];
  Tensor output = inplace ? a : newOutput(allocator, a.getDeviceType(), a.getDataType(), in[1].tensor.getShape());
  failFromContext(context, vl::accumulate(context, output, alpha, a, beta, b));
  if (!inplace) out[0] = output;
  (void)nout;
}

// ------------------------------------------------------------------------------------------ vl_nnloss
// matlab/vl_nnloss.m:129-317 (MATLAB code in the reference): (x, c [, dzdy], options)

// A single-precision device copy of a numeric argument that may live on the host (labels and instance weights come
// from the data loader there; the reference gathers the labels to the host, the kernels here want them on the device).
Tensor onDeviceAsSingle(Context& context, Allocator& allocator, Arg const& a, char const* NAME) {
  if (a.kind != Arg::Array) raise(VLE_IllegalArgument, std::string(NAME) + " is not a numeric array.");
  Tensor const& t = a.tensor;
  if (t.getDeviceType() == VLDT_GPU) {
    if (t.getDataType() != VLDT_Float) raise(VLE_Unsupported, std::string(NAME) + ": only SINGLE arrays are supported on the device.");
    return t;
  }
  const std::size_t n = t.getNumElements();
  std::vector<float> host(n);
  if (t.getDataType() == VLDT_Float) for (std::size_t i = 0; i < n; ++i) host[i] = ((float const*)t.getMemory())[i];
  else if (t.getDataType() == VLDT_Double) for (std::size_t i = 0; i < n; ++i) host[i] = (float)((double const*)t.getMemory())[i];
  else raise(VLE_IllegalArgument, std::string(NAME) + " is neither SINGLE nor DOUBLE.");
  Tensor copy = newOutput(allocator, VLDT_GPU, VLDT_Float, t.getShape());
  hipStream_t stream = (hipStream_t)context.getHipHelper().getStream();
  if (n && (hipMemcpyAsync(copy.getMemory(), host.data(), n * sizeof(float), hipMemcpyHostToDevice, stream) != hipSuccess ||
            hipStreamSynchronize(stream) != hipSuccess)) {
    (void)hipGetLastError();
    raise(VLE_Cuda, std::string(NAME) + ": could not be copied to the device.");
  }
  return copy;
}

void nnloss(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in) {
  enum { optLoss, optInstanceWeights, optClassWeights, optThreshold, optNormalise, optTopK };
  static OptionSpec const specs[] = {{"loss", true, optLoss}, {"instanceWeights", true, optInstanceWeights},
                                     {"classWeights", true, optClassWeights}, {"threshold", true, optThreshold},
                                     {"normalise", true, optNormalise}, {"topK", true, optTopK}, {NULL, false, 0}};
  static char const* const names[] = {"classerror", "topkerror", "log", "softmaxlog", "mhinge", "mshinge",
                                      "binaryerror", "binarylog", "logistic", "hinge"};
  if (nin < 2) raise(VLE_IllegalArgument, "There are less than two arguments.");
  int next = 2;
  Arg const* dzdy = NULL;
  if (nin > 2 && in[2].kind != Arg::String) {   // (vl_nnloss.m:129-134)
    dzdy = &in[2];
    next = 3;
  }
  mcn_loss_geom g;
  g.loss = MCN_LOSS_SOFTMAXLOG; g.topK = 5; g.normalise = 1; g.threshold = 0;   // (vl_nnloss.m:136-141)
  Arg const* weights = NULL;
  int opt;
  Arg const* value = NULL;
  auto scalar = [&](Arg const& a, char const* NAME) -> double {
    if (!(isPlainMatrix(a) && a.tensor.getNumElements() == 1)) raise(VLE_IllegalArgument, std::string(NAME) + " is not a plain scalar.");
    return values(a)[0];
  };
  while ((opt = nextOption(in, nin, specs, &next, &value)) >= 0) {
    switch (opt) {
      case optLoss: {
        if (value->kind != Arg::String) raise(VLE_IllegalArgument, "LOSS is not a string.");
        int k = 0;
        for (; k < 10; ++k) if (sameTextNoCase(value->text, names[k])) break;
        if (k == 10) raise(VLE_IllegalArgument, "Unknown loss '" + value->text + "'.");   // (vl_nnloss.m:199-200)
        g.loss = k;
        break;
      }
      case optInstanceWeights: if (!(value->kind == Arg::Array && value->tensor.getNumElements() == 0)) weights = value; break;
      case optClassWeights:
        if (!(value->kind == Arg::Array && value->tensor.getNumElements() == 0))
          raise(VLE_Unsupported, "CLASSWEIGHTS are not used by vl_nnloss.");   // (parsed and never read by the reference)
        break;
      case optThreshold: g.threshold = scalar(*value, "THRESHOLD"); break;
      case optNormalise: g.normalise = scalar(*value, "NORMALISE") != 0; break;
      case optTopK: g.topK = (int)scalar(*value, "TOPK"); break;
    }
  }
  Tensor x = dataTensor(in[0], "X", 4);
  if (x.getDeviceType() != VLDT_GPU) raise(VLE_Unsupported, "vl_nnloss: X is on the CPU; this library implements the GPU (HIP, gfx950) device only");
  if (x.getDataType() != VLDT_Float) raise(VLE_Unsupported, "vl_nnloss: only single precision is implemented on the HIP device");
  g.H = (int)x.getHeight(); g.W = (int)x.getWidth(); g.C = (int)x.getDepth(); g.N = (int)x.getSize();
  Tensor c = onDeviceAsSingle(context, allocator, in[1], "C");
  Tensor w;
  if (weights) w = onDeviceAsSingle(context, allocator, *weights, "INSTANCEWEIGHTS");
  void* stream = context.getHipHelper().getStream();
  const bool backMode = dzdy && !(dzdy->kind == Arg::Array && dzdy->tensor.getNumElements() == 0);
  int rc;
  if (!backMode) {
    const std::size_t bytes = mcn_loss_workspace_bytes(&g);
    void* ws = bytes ? context.getWorkspace(VLDT_GPU, bytes) : NULL;
    if (bytes && !ws) failFromContext(context, context.getLastError());
    std::size_t one[2] = {1, 1};
    Tensor y = newOutput(allocator, VLDT_GPU, VLDT_Float, TensorShape(one, 2));
    rc = mcn_loss_forward(stream, &g, (float*)y.getMemory(), (float const*)x.getMemory(), (float const*)c.getMemory(),
                          c.getNumElements(), (float const*)w.getMemory(), w.getNumElements(), ws, bytes);
    out[0] = y;
  } else {
    const double dz = scalar(*dzdy, "DZDY");
    Tensor dzdx = newOutput(allocator, VLDT_GPU, VLDT_Float, in[0].tensor.getShape());
    rc = mcn_loss_backward(stream, &g, (float*)dzdx.getMemory(), (float const*)x.getMemory(), (float const*)c.getMemory(),
                           c.getNumElements(), (float const*)w.getMemory(), w.getNumElements(), dz);
    out[0] = dzdx;
  }
  if (rc) raise(rc > 0 && rc <= (int)VLE_Interrupted ? (ErrorCode)rc : VLE_Unknown, mcn_last_error_message());
  (void)nout;
}

// ------------------------------------------------------------------------------------------ vl_nnrelu
// matlab/vl_nnrelu.m:33-55: (x [, dzdy], 'leak', value)

void nnrelu(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in) {
  enum { optLeak };
  static OptionSpec const specs[] = {{"leak", true, optLeak}, {NULL, false, 0}};
  if (nin < 1) raise(VLE_IllegalArgument, "There are no arguments.");
  int next = 1;
  Arg const* dzdyArg = NULL;
  if (nin > 1 && in[1].kind != Arg::String) {
    dzdyArg = &in[1];
    next = 2;
  }
  double leak = 0;
  int opt;
  Arg const* value = NULL;
  while ((opt = nextOption(in, nin, specs, &next, &value)) >= 0) {
    if (!(isPlainMatrix(*value) && value->tensor.getNumElements() == 1)) raise(VLE_IllegalArgument, "LEAK is not a plain scalar.");
    leak = values(*value)[0];
  }
  Tensor x = dataTensor(in[0], "X", 4);
  if (x.getDeviceType() != VLDT_GPU) raise(VLE_Unsupported, "vl_nnrelu: X is on the CPU; this library implements the GPU (HIP, gfx950) device only");
  if (x.getDataType() != VLDT_Float) raise(VLE_Unsupported, "vl_nnrelu: only single precision is implemented on the HIP device");
  void* stream = context.getHipHelper().getStream();
  Tensor y = newOutput(allocator, VLDT_GPU, VLDT_Float, in[0].tensor.getShape());
  const bool backMode = dzdyArg && !(dzdyArg->kind == Arg::Array && dzdyArg->tensor.getNumElements() == 0);
  int rc;
  if (!backMode) {
    rc = mcn_relu_forward_leaky(stream, (float*)y.getMemory(), (float const*)x.getMemory(), x.getNumElements(), leak);
  } else {
    Tensor dzdy = dataTensor(*dzdyArg, "DZDY", 4);
    if (!areCompatible(x, dzdy)) raise(VLE_IllegalArgument, "X and DZDY do not have compatible formats.");
    if (dzdy.getNumElements() != x.getNumElements()) raise(VLE_IllegalArgument, "X and DZDY do not have the same number of elements.");
    rc = mcn_relu_backward_leaky(stream, (float*)y.getMemory(), (float const*)x.getMemory(), (float const*)dzdy.getMemory(),
                                 x.getNumElements(), leak);
  }
  if (rc) raise(rc > 0 && rc <= (int)VLE_Interrupted ? (ErrorCode)rc : VLE_Unknown, mcn_last_error_message());
  out[0] = y;
  (void)nout;
}

// ------------------------------------------------------------------------------------------ vl_nnsoftmax
// matlab/vl_nnsoftmax.m:20-28: (x [, dzdy])

void nnsoftmax(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in) {
  if (nin < 1) raise(VLE_IllegalArgument, "There are no arguments.");
  if (nin > 2) raise(VLE_IllegalArgument, "There are more than two arguments.");
  Tensor x = dataTensor(in[0], "X", 4);
  if (x.getDeviceType() != VLDT_GPU) raise(VLE_Unsupported, "vl_nnsoftmax: X is on the CPU; this library implements the GPU (HIP, gfx950) device only");
  if (x.getDataType() != VLDT_Float) raise(VLE_Unsupported, "vl_nnsoftmax: only single precision is implemented on the HIP device");
  void* stream = context.getHipHelper().getStream();
  Tensor y = newOutput(allocator, VLDT_GPU, VLDT_Float, in[0].tensor.getShape());
  const int H = (int)x.getHeight(), W = (int)x.getWidth(), C = (int)x.getDepth(), N = (int)x.getSize();
  int rc;
  if (nin < 2) {
    rc = mcn_softmax_forward(stream, (float*)y.getMemory(), (float const*)x.getMemory(), H, W, C, N);
  } else {
    Tensor dzdy = dataTensor(in[1], "DZDY", 4);
    if (!areCompatible(x, dzdy)) raise(VLE_IllegalArgument, "X and DZDY do not have compatible formats.");
    if (dzdy.getNumElements() != x.getNumElements()) raise(VLE_IllegalArgument, "X and DZDY do not have the same number of elements.");
    rc = mcn_softmax_backward(stream, (float*)y.getMemory(), (float const*)x.getMemory(), (float const*)dzdy.getMemory(), H, W, C, N);
  }
  if (rc) raise(rc > 0 && rc <= (int)VLE_Interrupted ? (ErrorCode)rc : VLE_Unknown, mcn_last_error_message());
  out[0] = y;
  (void)nout;
}

typedef void (*Body)(Context&, Allocator&, int, Tensor*, int, Arg const*);

ErrorCode guarded(Body body, Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in,
                  std::string& message) {
  message.clear();
  context.resetLastError();
  try {
    body(context, allocator, nout, out, nin, in);
  } catch (Failure const& f) {
    message = f.text;
    return f.code;
  }
  return VLE_Success;
}

}  // namespace

ErrorCode vl_nnconv(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in, std::string& message) {
  return guarded(nnconv, context, allocator, nout, out, nin, in, message);
}
ErrorCode vl_nnconvt(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in, std::string& message) {
  return guarded(nnconvt, context, allocator, nout, out, nin, in, message);
}
ErrorCode vl_nnbnorm(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in, std::string& message) {
  return guarded(nnbnorm, context, allocator, nout, out, nin, in, message);
}
ErrorCode vl_nnpool(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in, std::string& message) {
  return guarded(nnpool, context, allocator, nout, out, nin, in, message);
}
ErrorCode vl_taccum(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in, std::string& message) {
  return guarded(taccum, context, allocator, nout, out, nin, in, message);
}
ErrorCode vl_nnsoftmax(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in, std::string& message) {
  return guarded(nnsoftmax, context, allocator, nout, out, nin, in, message);
}
ErrorCode vl_nnrelu(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in, std::string& message) {
  return guarded(nnrelu, context, allocator, nout, out, nin, in, message);
}
ErrorCode vl_nnloss(Context& context, Allocator& allocator, int nout, Tensor* out, int nin, Arg const* in, std::string& message) {
  return guarded(nnloss, context, allocator, nout, out, nin, in, message);
}

} }  // namespace vl::frontend
