// NativeOps boundary, part 5: the members of the reference's class that are outside the legacy op-execution path
// (graphs, custom ops, aggregates, meta-ops, sort, gradient compression, numpy and mmap helpers, host-side concat).
// They exist so that a binding generated from the reference's header resolves every symbol; none of them does the
// reference's work.  Each call prints one line naming the member and returns 0 / null / false.
// Reference declarations: blas/NativeOps.h (specialConcat*, execAggregate*, execMetaPredicate*, encode* / decode*,
// sort*, mmapFile, execute*Graph*, execCustomOp*, calculateOutputShapes*, ...).
#include <cstdio>

#include "../../include/NativeOps.h"

namespace {

void offPath(const char *member) { std::printf("NativeOps::%s is not on the legacy op path of this library: nothing done\n", member); }

}  // namespace

#define ND4J_OFFPATH_STUBS(SUFFIX, T, S)                                                                           \
    void NativeOps::specialConcat##SUFFIX(Nd4jPointer *, int, int, Nd4jPointer *, Nd4jPointer *, T *, Nd4jLong *,  \
                                          Nd4jPointer *, Nd4jPointer *) { offPath("specialConcat" #SUFFIX); }      \
    void NativeOps::execAggregate##SUFFIX(Nd4jPointer *, int, T **, int, Nd4jLong **, int, int *, int, int **, int, \
                                          T *, int) { offPath("execAggregate" #SUFFIX); }                          \
    void NativeOps::execAggregateBatch##SUFFIX(Nd4jPointer *, int, int, int, int, int, int, int, int, void *) {    \
        offPath("execAggregateBatch" #SUFFIX);                                                                     \
    }                                                                                                              \
    void NativeOps::execMetaPredicateStrided##SUFFIX(Nd4jPointer *, const int, const int, const int, const int,    \
                                                     Nd4jLong, T *, Nd4jLong, T *, Nd4jLong, T *, Nd4jLong, T *,   \
                                                     T *, S, S) { offPath("execMetaPredicateStrided" #SUFFIX); }   \
    void NativeOps::execMetaPredicateShape##SUFFIX(Nd4jPointer *, const int, const int, const int, const int,      \
                                                   Nd4jLong, T *, Nd4jLong *, T *, Nd4jLong *, T *, Nd4jLong *,    \
                                                   T *, T *, S, S) { offPath("execMetaPredicateShape" #SUFFIX); }  \
    Nd4jLong NativeOps::encodeBitmap##SUFFIX(Nd4jPointer *, T *, Nd4jLong, int *, float) {                         \
        offPath("encodeBitmap" #SUFFIX);                                                                           \
        return 0;                                                                                                  \
    }                                                                                                              \
    void NativeOps::decodeBitmap##SUFFIX(Nd4jPointer *, void *, Nd4jLong, T *) { offPath("decodeBitmap" #SUFFIX); } \
    void NativeOps::encodeThresholdP1##SUFFIX(Nd4jPointer *, T *, Nd4jLong, int *, float) {                        \
        offPath("encodeThresholdP1" #SUFFIX);                                                                      \
    }                                                                                                              \
    void NativeOps::encodeThresholdP3##SUFFIX(Nd4jPointer *, T *, int *, Nd4jLong, int *) {                        \
        offPath("encodeThresholdP3" #SUFFIX);                                                                      \
    }                                                                                                              \
    void NativeOps::decodeThreshold##SUFFIX(Nd4jPointer *, void *, Nd4jLong, T *) {                                \
        offPath("decodeThreshold" #SUFFIX);                                                                        \
    }                                                                                                              \
    void NativeOps::sort##SUFFIX(Nd4jPointer *, T *, Nd4jLong *, bool) { offPath("sort" #SUFFIX); }                \
    void NativeOps::sortTad##SUFFIX(Nd4jPointer *, T *, Nd4jLong *, int *, int, Nd4jLong *, Nd4jLong *, bool) {    \
        offPath("sortTad" #SUFFIX);                                                                                \
    }                                                                                                              \
    void NativeOps::sortCooIndices##SUFFIX(Nd4jPointer *, Nd4jLong *, T *, Nd4jLong, int) {                        \
        offPath("sortCooIndices" #SUFFIX);                                                                         \
    }                                                                                                              \
    Nd4jPointer NativeOps::executeFlatGraph##SUFFIX(Nd4jPointer *, Nd4jPointer) {                                  \
        offPath("executeFlatGraph" #SUFFIX);                                                                       \
        return nullptr;                                                                                            \
    }                                                                                                              \
    int NativeOps::execCustomOp##SUFFIX(Nd4jPointer *, Nd4jLong, Nd4jPointer *, Nd4jPointer *, int, Nd4jPointer *, \
                                        Nd4jPointer *, int, T *, int, Nd4jLong *, int, bool) {                     \
        offPath("execCustomOp" #SUFFIX);                                                                           \
        return 1; /* ND4J_STATUS_BAD_INPUT-class failure: nothing ran */                                           \
    }                                                                                                              \
    nd4j::ShapeList *NativeOps::calculateOutputShapes##SUFFIX(Nd4jPointer *, Nd4jLong, Nd4jPointer *, int, T *,    \
                                                              int, Nd4jLong *, int) {                              \
        offPath("calculateOutputShapes" #SUFFIX);                                                                  \
        return nullptr;                                                                                            \
    }                                                                                                              \
    nd4j::ShapeList *NativeOps::calculateOutputShapes##SUFFIX(Nd4jPointer *, Nd4jLong, Nd4jPointer *,              \
                                                              Nd4jPointer *, int, T *, int, Nd4jLong *, int) {     \
        offPath("calculateOutputShapes" #SUFFIX);                                                                  \
        return nullptr;                                                                                            \
    }                                                                                                              \
    int NativeOps::registerGraph##SUFFIX(Nd4jPointer *, Nd4jLong, Nd4jPointer) {                                   \
        offPath("registerGraph" #SUFFIX);                                                                          \
        return 1;                                                                                                  \
    }                                                                                                              \
    nd4j::graph::VariablesSet<T> *NativeOps::executeStoredGraph##SUFFIX(Nd4jPointer *, Nd4jLong, Nd4jPointer *,    \
                                                                        Nd4jPointer *, int *, int) {               \
        offPath("executeStoredGraph" #SUFFIX);                                                                     \
        return nullptr;                                                                                            \
    }                                                                                                              \
    void NativeOps::deleteVariablesSet##SUFFIX(Nd4jPointer) { offPath("deleteVariablesSet" #SUFFIX); }             \
    Nd4jPointer NativeOps::getGraphState##SUFFIX(Nd4jLong) {                                                       \
        offPath("getGraphState" #SUFFIX);                                                                          \
        return nullptr;                                                                                            \
    }                                                                                                              \
    void NativeOps::deleteGraphState##SUFFIX(Nd4jPointer) { offPath("deleteGraphState" #SUFFIX); }                 \
    Nd4jStatus NativeOps::execCustomOpWithScope##SUFFIX(Nd4jPointer *, Nd4jPointer, Nd4jLong, Nd4jLong *, int,     \
                                                        Nd4jPointer *, Nd4jPointer *, int, Nd4jPointer *,          \
                                                        Nd4jPointer *, int) {                                      \
        offPath("execCustomOpWithScope" #SUFFIX);                                                                  \
        return 1;                                                                                                  \
    }

ND4J_OFFPATH_STUBS(Float, float, float)
ND4J_OFFPATH_STUBS(Half, float16, float)
ND4J_OFFPATH_STUBS(Double, double, double)

void NativeOps::execMetaPredicateReduceFloat(Nd4jPointer *, const int, const int, const int, const int, float *, Nd4jLong *,
                                             float *, Nd4jLong *, float *, Nd4jLong *, int *, int, Nd4jLong *, Nd4jLong *,
                                             float *, float *, float, float, bool) {
    offPath("execMetaPredicateReduceFloat");
}
void NativeOps::encodeThresholdP2Int(Nd4jPointer *, int *, Nd4jLong, int *) { offPath("encodeThresholdP2Int"); }
Nd4jPointer NativeOps::executeProtoGraphFloat(Nd4jPointer *, Nd4jPointer) {
    offPath("executeProtoGraphFloat");
    return nullptr;
}
Nd4jPointer NativeOps::executeProtoGraphFloat(Nd4jPointer *, const char *) {
    offPath("executeProtoGraphFloat");
    return nullptr;
}
// cuBLAS / cuSOLVER function pointers of the reference's BlasHelper: nothing here calls them
void NativeOps::initializeFunctions(Nd4jPointer *) {}
// one GPU per process: there is no peer to enable
void NativeOps::enableP2P(bool) {}
void NativeOps::checkP2P() {}
bool NativeOps::isP2PAvailable() { return false; }
bool NativeOps::isExperimentalEnabled() { return false; }
Nd4jPointer NativeOps::shapeBufferForNumpy(Nd4jPointer) {
    offPath("shapeBufferForNumpy");
    return nullptr;
}
Nd4jPointer NativeOps::dataPointForNumpy(Nd4jPointer) {
    offPath("dataPointForNumpy");
    return nullptr;
}
Nd4jPointer NativeOps::numpyFromFile(std::string) {
    offPath("numpyFromFile");
    return nullptr;
}
void NativeOps::releaseNumpy(Nd4jPointer) { offPath("releaseNumpy"); }
// shape::shapeInfoLength of a host shapeInfo buffer: 2 * rank + 4 (blas/NativeOps.h: lengthForShapeBufferPointer)
int NativeOps::lengthForShapeBufferPointer(Nd4jPointer buffer) {
    if (buffer == nullptr) return 0;
    return (int)(2 * reinterpret_cast<Nd4jLong *>(buffer)[0] + 4);
}
int NativeOps::elementSizeForNpyArray(Nd4jPointer) {
    offPath("elementSizeForNpyArray");
    return 0;
}
Nd4jPointer NativeOps::pointerForAddress(Nd4jLong address) { return reinterpret_cast<Nd4jPointer>(address); }
Nd4jLong *NativeOps::mmapFile(Nd4jPointer *, const char *, Nd4jLong) {
    offPath("mmapFile");
    return nullptr;
}
void NativeOps::munmapFile(Nd4jPointer *, Nd4jLong *, Nd4jLong) { offPath("munmapFile"); }
const char *NativeOps::getAllCustomOps() { return ""; }
const char *NativeOps::getAllOperations() { return ""; }
void NativeOps::deleteShapeList(Nd4jPointer) { offPath("deleteShapeList"); }
int NativeOps::unregisterGraph(Nd4jPointer *, Nd4jLong) {
    offPath("unregisterGraph");
    return 1;
}
void NativeOps::deleteIntArray(Nd4jPointer pointer) { delete[] reinterpret_cast<int *>(pointer); }
void NativeOps::deleteLongArray(Nd4jPointer pointer) { delete[] reinterpret_cast<Nd4jLong *>(pointer); }
void NativeOps::deletePointerArray(Nd4jPointer pointer) { delete[] reinterpret_cast<Nd4jPointer *>(pointer); }
