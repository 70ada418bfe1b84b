// Notes about rulebooks built on a handle: which pair tensors came from
// mluOpGetIndicePairs, and whether their input rows were in cell order.
#include "sparse_conv/rulebook_notes.h"

namespace mluop {
namespace sparse_conv {

RulebookReportTarget openRulebookNote(mluOpContext *handle, const void *pairs, int K, int L) {
  // an older note about the same address describes a tensor that is being overwritten
  for (auto &n : handle->rulebook_notes)
    if (n.pairs == pairs) n.pairs = nullptr;
  const int slot = handle->next_rulebook_note;
  handle->next_rulebook_note = (slot + 1) % mluOpContext::kRulebookNotes;
  mluOpContext::RulebookNote &note = handle->rulebook_notes[slot];
  note.pairs = pairs;
  note.K = K;
  note.L = L;
  note.stamp = handle->next_stamp++;
  // the device ORs its flags into a cleared word and stores the stamp last
  handle->rulebook_reports[slot].stamp = 0;
  handle->rulebook_reports[slot].rows_in_order = 0;
  RulebookReportTarget t;
  t.stamp = note.stamp;
  // A captured rulebook files no report in host memory: nothing runs now, so no report of
  // this call could arrive, and a replay must not write into a slot that by then belongs to
  // another rulebook (or to a handle that is gone).
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(handle->queue, &capturing) != hipSuccess) (void)hipGetLastError();
  if (capturing == hipStreamCaptureStatusNone) {
    t.stamp_word = &handle->rulebook_reports[slot].stamp;
    t.order_word = &handle->rulebook_reports[slot].rows_in_order;
  }
  return t;
}

void consultRulebookNotes(mluOpContext *handle, int row_column, ConvProblem *p) {
  p->ticket = handle->next_stamp++;
  p->list_trust = ListTrust::kNone;
  if (handle->rulebook_reports == nullptr) return;
  for (int slot = 0; slot < mluOpContext::kRulebookNotes; ++slot) {
    const mluOpContext::RulebookNote &note = handle->rulebook_notes[slot];
    if (note.pairs != p->indice_pairs || note.K != p->K || note.L != p->L) continue;
    if (row_column == 0) {
      p->list_trust = ListTrust::kInOrder;
      return;
    }
    const volatile mluOpContext::RulebookReport *report = &handle->rulebook_reports[slot];
    if (__atomic_load_n(&report->stamp, __ATOMIC_ACQUIRE) != note.stamp) {
      // not arrived (or never sent: a captured rulebook files none)
      p->list_trust = ListTrust::kUnknown;
      return;
    }
    p->list_trust = report->rows_in_order != 0 ? ListTrust::kInOrder : ListTrust::kNone;
    return;
  }
}

void forgetRulebookNotesIn(mluOpContext *handle, const void *out, size_t bytes) {
  const char *lo = static_cast<const char *>(out);
  for (auto &n : handle->rulebook_notes) {
    const char *at = static_cast<const char *>(n.pairs);
    if (at != nullptr && at >= lo && at < lo + bytes) n.pairs = nullptr;
  }
}

}  // namespace sparse_conv
}  // namespace mluop
