// NNDefs.h — engine-wide constants and enumerations (the reference keeps them at the top of engine/NNTypes.h:45-133).
// Ordinals are stored in network files and must not change.
#ifndef DSSTNE_AMD_NNDEFS_H
#define DSSTNE_AMD_NNDEFS_H

#include "GpuTypes.h"

static const float NN_VERSION = 0.9f;
static const float MAX_VALUE = 999999999999999.0f;   // engine/NNTypes.h:49: top-K sentinel magnitude

enum { DefaultBatch = 512 };

enum Mode { Prediction = 0, Training = 1, Validation = 2, Unspecified = 3 };

enum TrainingMode { SGD = 0, Momentum = 1, AdaGrad = 2, Nesterov = 3, RMSProp = 4, AdaDelta = 5, Adam = 6 };

enum ErrorFunction { L1, L2, CrossEntropy, ScaledMarginalCrossEntropy, DataScaledMarginalCrossEntropy, Hinge, L2Hinge };

// ordinals are stored in network files (engine/NNTypes.h:91-105)
enum Activation {
    Sigmoid,
    Tanh,
    RectifiedLinear,
    Linear,
    ParametricRectifiedLinear,
    SoftPlus,
    SoftSign,
    SoftMax,
    RELUMax,
    LinearMax,
    ExponentialLinear,
    LeakyRectifiedLinear,
    ScaledExponentialLinear,
};

enum WeightInitialization { Xavier, CaffeXavier, Gaussian, Uniform, UnitBall, Constant, SELU };

enum PoolingFunction { None, Max, Average, LRN, Maxout, DotProduct, Cosine, Stochastic, LCN, GlobalTemporal };

ostream& operator<<(ostream& out, const Activation& a);

#endif
