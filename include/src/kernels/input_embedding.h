// launchInputEmbedding -- same declaration as the reference's src/kernels/input_embedding.h:6-9.
// output [tokens, hidden] = embed_table->data[input_ids[t], :]; throws if the token counts differ.
// If embed_table->shape holds {vocab, hidden} the ids are bounds-checked (out-of-range -> zero row).
#pragma once
#include "src/utils/tensor.h"
#include "src/weights/llama/embedding_weights.h"
template <typename T>
void launchInputEmbedding(TensorWrapper<int>* input_ids, TensorWrapper<T>* output,
                          EmbeddingWeight<T>* embed_table);
