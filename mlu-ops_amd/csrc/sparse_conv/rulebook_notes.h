// What a handle remembers about the rulebooks it built (mluOpContext::rulebook_notes).
#ifndef MLUOP_AMD_SPARSE_CONV_RULEBOOK_NOTES_H_
#define MLUOP_AMD_SPARSE_CONV_RULEBOOK_NOTES_H_

#include "core/core.h"
#include "sparse_conv/indice_conv.h"
#include "sparse_conv/rulebook.h"

namespace mluop {
namespace sparse_conv {

// Takes a note for the rulebook about to be written to `pairs` and returns where its last
// kernel reports to.
RulebookReportTarget openRulebookNote(mluOpContext *handle, const void *pairs, int K, int L);

// Sets p->list_trust and p->ticket for a forward / backward-data launch whose result rows
// are named by pair column `row_column`.  Column 0 of a rulebook this handle built ascends by
// construction; column 1 does when the report says the input rows were in cell order.  A
// report that has not arrived yet leaves the question to the kernels.
void consultRulebookNotes(mluOpContext *handle, int row_column, ConvProblem *p);

// Memory [out, out + bytes) is about to be written by an operator of this handle: a note about
// a pair tensor that starts inside it describes memory that was handed out again, and is dropped.
void forgetRulebookNotesIn(mluOpContext *handle, const void *out, size_t bytes);

}  // namespace sparse_conv
}  // namespace mluop

#endif  // MLUOP_AMD_SPARSE_CONV_RULEBOOK_NOTES_H_
