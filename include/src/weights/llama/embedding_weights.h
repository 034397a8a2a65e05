// Token-embedding table, [vocab, hidden] row-major on the device, as `data` of a BaseWeight.
// Same type as the reference's src/weights/llama/embedding_weights.h.  launchInputEmbedding reads
// `data`; if `shape` holds {vocab, hidden} it also bounds-checks the token ids against `vocab`
// (the reference never looks at `shape`, so leaving it empty reproduces its unchecked gather).
#pragma once
#include "src/weights/base_weights.h"

template <typename T>
struct EmbeddingWeight : public BaseWeight<T> {};
