// qed_builder.h -- text tables -> QED file, the job of the reference's EmbeddingBuilder
// (blaze/store/quick_embedding/embedding_builder.cc:20-255, exported as Blaze_QuickEmbeddingBuildFp32/Fp16).
// Input: `path/meta` lists one table file name per line (a last line without a newline is dropped, as the
// reference's ParseMeta does, :57-75); each table file holds lines `key,w0,...,w(dim-1)` (dim = fields of the
// first line - 1, lines with another field count are skipped).  Output: the file layout described in
// qed_store.h, table i under gid i.  The pad byte at offset 0 of each weight blob is written as zero.
#pragma once

#include <string>

namespace blaze {
namespace store {

bool BuildQuickEmbedding(const std::string& path, const std::string& meta, const std::string& output_file, int value_type,
                         int thread_num, std::string* err);

}  // namespace store
}  // namespace blaze
