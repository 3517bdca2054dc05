// efanna2e::Index -- the abstract index the reference's IndexGPU derives from
// (include/efanna2e/index.h:20-64, src/index.cpp:9-29), so that code written
// against the reference's class hierarchy (an Index* handed to IndexGPU's
// constructor, calls through the base pointer) compiles against this library.
//
// The reference's constructor also allocates a host-side Distance object
// (DistanceL2 / DistanceInnerProduct, AVX-512 code of efanna2e/distance.h) and
// prints which one; nothing on this library's path measures distances on the
// host, so distance_ stays null here and nothing is printed.
#pragma once
#include <cstddef>

#include "../coral_search.h"
#include "parameters.h"

namespace efanna2e {

enum Metric { L2 = 0, INNER_PRODUCT = 1, FAST_L2 = 2, PQ = 3, COSINE = 4 };  // efanna2e/distance.h:15

class Distance;  // efanna2e/distance.h:16-20; never instantiated by this library

class CORAL_API Index {
   public:
    explicit Index(const size_t dimension, const size_t n, Metric metric);
    virtual ~Index();

    virtual void Build(size_t n, const float* data, const Parameters& parameters) = 0;
    virtual void Search(const float* query, const float* x, size_t k, const Parameters& parameters,
                        unsigned* indices, float* res_dists) = 0;
    virtual void Save(const char* filename) = 0;
    virtual void Load(const char* filename) = 0;

    inline bool HasBuilt() const { return has_built; }
    inline size_t GetDimension() const { return dimension_; }
    inline size_t GetSizeOfDataset() const { return nd_; }
    inline const float* GetDataset() const { return data_; }
    inline const float* GetSampledQuerySet() const { return data_sq_; }
    inline const float* GetBasePointSet() const { return data_bp_; }

   protected:
    const size_t dimension_;
    const float* data_ = nullptr;
    float* data_sq_ = nullptr;
    float* data_bp_ = nullptr;
    size_t nd_;
    size_t nd_sq_ = 0;
    bool has_built = false;
    bool bipartite_ = false;
    Distance* distance_ = nullptr;
    Metric metric_;
};

}  // namespace efanna2e
