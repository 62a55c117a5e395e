// Reconstruct a serialized object from its recorded type name (reference: include/bb/ObjectLoader.h:407-447
// `Object_Load` / `Object_LoadFromFile`).  Known here: the LUT layers of widths 2..6 on fp32 or packed-bit frames,
// BinaryLut6, StochasticBatchNormalization, AverageLut, MaxLut, Reduce, Binarize, HardTanh, RealToBinary, BinaryToReal, BinaryModulation, DifferentiableLutDiscreteN (the LUT layer put together from its parts), MaxPooling, UpSampling, Shuffle, the convolution wrapper with its Im2Col / Col2Im, the layer list, and tensors.  An unknown name yields an empty pointer, as in the reference.
#pragma once

#include "bb/StochasticLutN.h"
#include "bb/DifferentiableLutN.h"
#include "bb/BinaryLutN.h"
#include "bb/ConvolutionIm2Col.h"
#include "bb/ConvolutionCol2Im.h"
#include "bb/Convolution2d.h"
#include "bb/Sequential.h"
#include "bb/StochasticBatchNormalization.h"
#include "bb/MaxLut.h"
#include "bb/AverageLut.h"
#include "bb/Reduce.h"
#include "bb/Binarize.h"
#include "bb/HardTanh.h"
#include "bb/RealToBinary.h"
#include "bb/BinaryToReal.h"
#include "bb/BinaryModulation.h"
#include "bb/DifferentiableLutDiscreteN.h"
#include "bb/MaxPooling.h"
#include "bb/UpSampling.h"
#include "bb/Shuffle.h"

namespace bb {

namespace detail {

template <int N>
inline std::shared_ptr<Object> CreateLutByName(std::string const &name)
{
    if (name == StochasticLutN<N, float, float>::ObjectName())     { return StochasticLutN<N, float, float>::Create((index_t)1); }
    if (name == StochasticLutN<N, Bit, float>::ObjectName())       { return StochasticLutN<N, Bit, float>::Create((index_t)1); }
    if (name == DifferentiableLutN<N, float, float>::ObjectName()) { return DifferentiableLutN<N, float, float>::Create((index_t)1); }
    if (name == DifferentiableLutN<N, Bit, float>::ObjectName())   { return DifferentiableLutN<N, Bit, float>::Create((index_t)1); }
    if (name == DifferentiableLutDiscreteN<N, float, float>::ObjectName()) { return DifferentiableLutDiscreteN<N, float, float>::Create((index_t)1); }
    if (name == DifferentiableLutDiscreteN<N, Bit, float>::ObjectName())   { return DifferentiableLutDiscreteN<N, Bit, float>::Create((index_t)1); }
    return std::shared_ptr<Object>();
}

inline std::shared_ptr<Object> CreateByName(std::string const &name)
{
    if (name == "Tensor")       { return std::make_shared<Tensor>(); }
    if (name == "Tensor_fp32")  { return std::make_shared<Tensor_<float>>(); }
    if (name == "Tensor_fp64")  { return std::make_shared<Tensor_<double>>(); }
    if (name == "Tensor_int32") { return std::make_shared<Tensor_<std::int32_t>>(); }
    if (name == BinaryLutN<6, Bit, float>::ObjectName()) { return BinaryLutN<6, Bit, float>::Create((index_t)1); }
    if (name == BinaryLutN<5, Bit, float>::ObjectName()) { return BinaryLutN<5, Bit, float>::Create((index_t)1); }
    if (name == BinaryLutN<4, Bit, float>::ObjectName()) { return BinaryLutN<4, Bit, float>::Create((index_t)1); }
    if (name == BinaryLutN<3, Bit, float>::ObjectName()) { return BinaryLutN<3, Bit, float>::Create((index_t)1); }
    if (name == BinaryLutN<2, Bit, float>::ObjectName()) { return BinaryLutN<2, Bit, float>::Create((index_t)1); }
    if (name == Sequential::ObjectName())                         { return Sequential::Create(); }
    if (name == StochasticBatchNormalization<float>::ObjectName()) { return StochasticBatchNormalization<float>::Create(); }
    if (name == AverageLut<float, float>::ObjectName())           { return AverageLut<float, float>::Create(); }
    if (name == AverageLut<Bit, float>::ObjectName())             { return AverageLut<Bit, float>::Create(); }
    if (name == MaxLut<float, float>::ObjectName())               { return MaxLut<float, float>::Create(); }
    if (name == Reduce<float, float>::ObjectName())               { return Reduce<float, float>::Create(); }
    if (name == Reduce<Bit, float>::ObjectName())                 { return Reduce<Bit, float>::Create(); }
    if (name == MaxLut<Bit, float>::ObjectName())                 { return MaxLut<Bit, float>::Create(); }
    if (name == Binarize<float, float>::ObjectName())             { return Binarize<float, float>::Create(); }
    if (name == Binarize<Bit, float>::ObjectName())               { return Binarize<Bit, float>::Create(); }
    if (name == HardTanh<float, float>::ObjectName())             { return HardTanh<float, float>::Create(); }
    if (name == HardTanh<Bit, float>::ObjectName())               { return HardTanh<Bit, float>::Create(); }
    if (name == RealToBinary<float, float>::ObjectName())         { return RealToBinary<float, float>::Create(); }
    if (name == RealToBinary<Bit, float>::ObjectName())           { return RealToBinary<Bit, float>::Create(); }
    if (name == BinaryToReal<float, float>::ObjectName())         { return BinaryToReal<float, float>::Create(); }
    if (name == BinaryToReal<Bit, float>::ObjectName())           { return BinaryToReal<Bit, float>::Create(); }
    if (name == BinaryModulation<float, float>::ObjectName())     { return BinaryModulation<float, float>::Create(); }
    if (name == BinaryModulation<Bit, float>::ObjectName())       { return BinaryModulation<Bit, float>::Create(); }
    if (name == MaxPooling<float, float>::ObjectName())           { return MaxPooling<float, float>::Create(); }
    if (name == MaxPooling<Bit, float>::ObjectName())             { return MaxPooling<Bit, float>::Create(); }
    if (name == UpSampling<float, float>::ObjectName())           { return UpSampling<float, float>::Create(); }
    if (name == UpSampling<Bit, float>::ObjectName())             { return UpSampling<Bit, float>::Create(); }
    if (name == Shuffle::ObjectName())                            { return Shuffle::Create(); }
    if (name == Convolution2d<float, float>::ObjectName())        { return Convolution2d<float, float>::Create(); }
    if (name == Convolution2d<Bit, float>::ObjectName())          { return Convolution2d<Bit, float>::Create(); }
    if (name == ConvolutionIm2Col<float, float>::ObjectName())    { return ConvolutionIm2Col<float, float>::Create(1, 1); }
    if (name == ConvolutionIm2Col<Bit, float>::ObjectName())      { return ConvolutionIm2Col<Bit, float>::Create(1, 1); }
    if (name == ConvolutionCol2Im<float, float>::ObjectName())    { return ConvolutionCol2Im<float, float>::Create(); }
    if (name == ConvolutionCol2Im<Bit, float>::ObjectName())      { return ConvolutionCol2Im<Bit, float>::Create(); }
    std::shared_ptr<Object> obj;
    if ((obj = CreateLutByName<6>(name))) { return obj; }
    if ((obj = CreateLutByName<5>(name))) { return obj; }
    if ((obj = CreateLutByName<4>(name))) { return obj; }
    if ((obj = CreateLutByName<3>(name))) { return obj; }
    if ((obj = CreateLutByName<2>(name))) { return obj; }
    return obj;
}

}  // namespace detail

inline std::shared_ptr<Object> Object_Load(std::istream &is)
{
    std::string const name = Object::ReadHeader(is);
    std::shared_ptr<Object> obj = detail::CreateByName(name);
    if (obj) { obj->LoadObjectData(is); }
    return obj;
}

inline std::shared_ptr<Object> Object_LoadFromFile(std::string filename)
{
    std::ifstream ifs(filename, std::ios::binary);
    if (!ifs.is_open()) { return std::shared_ptr<Object>(); }
    return Object_Load(ifs);
}

}  // namespace bb
