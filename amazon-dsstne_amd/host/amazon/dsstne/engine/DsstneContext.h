// Callers of the reference include the context under engine/ (java/src/test/native/main.cpp:27); it lives in runtime/.
#include "amazon/dsstne/runtime/DsstneContext.h"
