// Does a plan compute exactly the decode + score filter of a YOLO-style detection head
// (fx_head.h)?  The lowered programs are compared with the programs this library lowers that
// computation to, instruction by instruction, after a normalisation that removes what may
// differ between two such regions: the numbering of the pointer slots, the order in which the
// output programs lie in the class, the number of classes C (row length 5 + C of the
// prediction tensor), the offsets per task and the threshold.  Everything else (operations,
// flags, immediates, temporaries, jump distances, the offset of every load inside its row)
// enters a hash that must equal the one of the reference lowering; a region that differs in any
// of it, or a change of the lowering itself, simply keeps the generic kernels.
#include <cstring>
#include <map>

#include "fx_lower.h"

namespace fx {

namespace {

struct Hasher {
  uint64_t h = 1469598103934665603ull;
  void mix(uint64_t v) {
    for (int i = 0; i < 8; ++i) {
      h ^= (v >> (8 * i)) & 0xffu;
      h *= 1099511628211ull;
    }
  }
};

// hash of the normalised programs of the reference lowering (tests/test_head_stream.py holds the
// region that must match it)
const uint64_t kHeadHash = FX_HEAD_NORM_HASH;

}  // namespace

void match_head(Plan* P) {
  FxHeadInfo& hi = P->head;
  hi = FxHeadInfo();
  const uint32_t* sb = P->blob.data();
  if (P->blob.size() < sizeof(FxHeader) / 4) return;
  const FxHeader* h = (const FxHeader*)sb;
  if (h->mode != FX_MODE_COMPACT || h->n_classes != 1) return;
  const FxClass& cl = *(const FxClass*)(sb + h->off_class);
  if (cl.n_outs != 3 || cl.n_tasks != h->n_tasks || cl.n_rows == 0) return;
  const uint32_t* taskmap = sb + h->off_taskmap;
  for (uint32_t t = 0; t < cl.n_tasks; ++t)
    if (taskmap[cl.first_task + t] != t) return;
  const FxInsn* ins = (const FxInsn*)(sb + cl.off_insn);
  const FxAffine* aff = (const FxAffine*)(sb + cl.off_aff);
  const FxOut* outs = (const FxOut*)(sb + cl.off_outs);
  // the output table is sorted by row length: objectness [K], boxes [K, 4], class scores [K, C]
  const FxOut &o_obj = outs[0], &o_box = outs[1], &o_cls = outs[2];
  if (o_obj.rank != 1 || o_obj.rowlen != 1) return;
  if (o_box.rank != 2 || o_box.rowlen != 4 || o_box.inner != 4) return;
  if (o_cls.rank != 2 || o_cls.rowlen < 4 || o_cls.rowlen % 4 != 0 || o_cls.inner != o_cls.rowlen) return;
  for (int k = 0; k < 3; ++k)
    if (outs[k].dtype != FX_F32 || outs[k].vt != FX_VT_F) return;
  const uint32_t C = o_cls.rowlen, S = C + 5;

  Hasher hs;
  // pointer slot -> buffer in order of first use: predictions, anchors, strides; with folded anchors
  // predictions, half sizes, strides, centres
  std::map<int32_t, int> buf_class;
  int32_t slot_of[4] = {0, 0, 0, 0}, tcoef_of[4] = {0, 0, 0, 0}, coef0_of[4] = {0, 0, 0, 0};
  bool bad = false;
  uint32_t thr_bits = 0;
  auto walk = [&](uint32_t pb, uint32_t pe, bool is_mask) {
    hs.mix(0xABCDull);
    hs.mix(pe - pb);
    for (uint32_t pc = pb; pc < pe && !bad; ++pc) {
      const FxInsn& x = ins[pc];
      hs.mix(x.op);
      hs.mix(x.flags);
      hs.mix(x.dt);
      const bool load = x.op == FX_LDA || x.op == FX_LDB || (x.flags & FX_F_MEMB) != 0;
      if (load) {
        auto it = buf_class.find(x.a);
        int bc;
        if (it == buf_class.end()) {
          bc = (int)buf_class.size();
          if (bc >= 4) { bad = true; return; }
          buf_class[x.a] = bc;
          slot_of[bc] = x.a;
          tcoef_of[bc] = aff[x.b].tcoef;
          coef0_of[bc] = fx_aff_coef(&aff[x.b], 0);
        } else {
          bc = it->second;
        }
        const FxAffine& a = aff[x.b];
        if (a.tcoef != tcoef_of[bc] || a.rcoef[0] != 0 || a.rcoef[1] != 0) { bad = true; return; }
        // the row stride of each buffer is fixed by its role (checked below, once the form is known)
        if (fx_aff_coef(&a, 0) != coef0_of[bc]) { bad = true; return; }
        hs.mix((uint64_t)bc);
        for (int k = 1; k < FX_MAXR; ++k) hs.mix((uint64_t)(uint32_t)fx_aff_coef(&a, k));
        hs.mix((uint64_t)(uint32_t)a.base);
        hs.mix(x.imm);
      } else if (x.op == FX_MIFR) {
        const FxAffine& a = aff[x.b];
        hs.mix((uint64_t)(uint32_t)(x.a - (int32_t)pb));
        for (int k = 0; k < FX_MAXR; ++k) hs.mix((uint64_t)(uint32_t)fx_aff_coef(&a, k));
        hs.mix((uint64_t)(uint32_t)a.tcoef);
        hs.mix((uint64_t)(uint32_t)a.base);
        hs.mix((uint64_t)(uint32_t)a.rcoef[0]);
        hs.mix((uint64_t)(uint32_t)a.rcoef[1]);
        hs.mix(x.imm);
      } else if (x.op == FX_MIF || x.op == FX_MELSE || x.op == FX_RNEXT) {
        hs.mix((uint64_t)(uint32_t)(x.a - (int32_t)pb));
        hs.mix((uint64_t)(uint32_t)x.b);
        hs.mix(x.imm);
      } else {
        hs.mix((uint64_t)(uint32_t)x.a);
        hs.mix((uint64_t)(uint32_t)x.b);
        if (is_mask && x.op == FX_FGE && (x.flags & FX_F_IMM)) thr_bits = x.imm;   // the threshold is a parameter
        else hs.mix(x.imm);
      }
    }
  };
  walk(cl.mask_begin, cl.mask_end, true);
  hs.mix(cl.mask_vt);
  for (int k = 0; k < 3 && !bad; ++k) {
    hs.mix(outs[k].lead);
    hs.mix(outs[k].pure);
    walk(outs[k].prog_begin, outs[k].prog_end, false);
  }
  hi.norm_hash = hs.h;
  if (bad) return;
  const bool plain = buf_class.size() == 3 && hs.h == kHeadHash && coef0_of[0] == (int32_t)S && coef0_of[1] == 4 &&
                     coef0_of[2] == 1;
  const bool folded = buf_class.size() == 4 && hs.h == FX_HEAD_NORM_HASH_FOLDED && coef0_of[0] == (int32_t)S &&
                      coef0_of[1] == 2 && coef0_of[2] == 1 && coef0_of[3] == 2;
  if (!plain && !folded) return;
  // 32-bit addressing of the kernel: checked for the prediction tensor by the plan already
  // (every buffer of a region lies below 4 GiB)
  hi.pred_slot = (uint32_t)slot_of[0];
  hi.strd_slot = (uint32_t)slot_of[2];
  hi.pred_tcoef = tcoef_of[0];
  hi.strd_tcoef = tcoef_of[2];
  hi.folded = folded;
  if (folded) {
    hi.half_slot = (uint32_t)slot_of[1];
    hi.half_tcoef = tcoef_of[1];
    hi.anc_slot = (uint32_t)slot_of[3];
    hi.anc_tcoef = tcoef_of[3];
  } else {
    hi.anc_slot = (uint32_t)slot_of[1];
    hi.anc_tcoef = tcoef_of[1];
  }
  hi.S = S;
  hi.C = C;
  hi.thr_bits = thr_bits;
  hi.n_rows = cl.n_rows;
  hi.n_tasks = cl.n_tasks;
  for (int k = 0; k < 3; ++k) {
    hi.out_slot[k] = outs[k].ptr_slot;
    hi.out_tstride[k] = outs[k].task_stride;
  }
  hi.slot_total = h->slot_total;
  hi.ok = true;
}

}  // namespace fx
