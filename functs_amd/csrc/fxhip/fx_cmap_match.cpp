// Does a plan compute exactly the decode + per-class score filter of an SSD-style detection head
// (fx_cmap.h)?  As in fx_head_match.cpp the lowered programs are compared with the programs this
// library lowers that computation to after a normalisation that removes what may differ between
// two such regions: the numbering of the pointer slots, the number of classes C (row length of
// the score tensor and extent of the two reductions), the first class, the threshold and the two
// variances.  Everything else enters a hash that must equal the one of the reference lowering.
#include <cstring>
#include <map>
#include <vector>

#include "fx_cmap.h"
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

// hash of the normalised programs of the reference lowering (tests/test_classmap_head.py holds the
// region that must match it)
const uint64_t kCmapHash = FX_CMAP_NORM_HASH;

}  // namespace

void match_classmap(Plan* P) {
  FxCmapInfo& ci = P->cmap;
  ci = FxCmapInfo();
  const uint32_t* sb = P->blob.data();
  if (P->blob.size() < sizeof(FxHeader) / 4) return;
  const FxHeader* h = (const FxHeader*)sb;
  if (h->mode != FX_MODE_COMPACT || h->n_classes != 1) return;
  const FxClass& cl = *(const FxClass*)(sb + h->off_class);
  if (cl.n_outs != 2 || cl.n_tasks != h->n_tasks || cl.n_rows == 0 || cl.n_tasks > FX_CMAP_MAX_TASKS) return;
  const uint32_t* taskmap = sb + h->off_taskmap;
  for (uint32_t t = 0; t < cl.n_tasks; ++t)
    if (taskmap[cl.first_task + t] != t) return;
  const FxInsn* ins = (const FxInsn*)(sb + cl.off_insn);
  const FxAffine* aff = (const FxAffine*)(sb + cl.off_aff);
  const FxOut* outs = (const FxOut*)(sb + cl.off_outs);
  // the output table is sorted by row length: scores [K], boxes [K, 4]
  const FxOut &o_sc = outs[0], &o_box = outs[1];
  if (o_sc.rank != 1 || o_sc.rowlen != 1) return;
  if (o_box.rank != 2 || o_box.rowlen != 4 || o_box.inner != 4) return;
  for (int k = 0; k < 2; ++k)
    if (outs[k].dtype != FX_F32 || outs[k].vt != FX_VT_F) return;

  Hasher hs;
  std::map<int32_t, int> buf_class;   // pointer slot -> 0 (scores), 1 (offsets), 2 (priors), in order of first use
  int32_t slot_of[3] = {0, 0, 0};
  bool bad = false;
  uint32_t thr_bits = 0, C = 0;
  int32_t first = -1;
  std::vector<uint32_t> var;          // immediates of the multiplications of the box program, in order
  auto mix_affine = [&](const FxAffine& a) {
    for (int k = 0; k < FX_MAXR; ++k) hs.mix((uint64_t)(uint32_t)fx_aff_coef(&a, k));
    hs.mix((uint64_t)(uint32_t)a.tcoef);
    hs.mix((uint64_t)(uint32_t)a.base);
    hs.mix((uint64_t)(uint32_t)a.rcoef[0]);
    hs.mix((uint64_t)(uint32_t)a.rcoef[1]);
  };
  auto walk = [&](uint32_t pb, uint32_t pe, int which) {   // 0 mask, 1 scores, 2 boxes
    hs.mix(0xC1A5ull);
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
          if (bc >= 3) { bad = true; return; }
          buf_class[x.a] = bc;
          slot_of[bc] = x.a;
        } else {
          bc = it->second;
        }
        const FxAffine& a = aff[x.b];
        hs.mix((uint64_t)bc);
        if (bc == 0) {
          // score rows of C floats: walked by a reduction (r = 1, no offset), or one column per task
          if (C == 0 || fx_aff_coef(&a, 0) != (int32_t)C) { bad = true; return; }
          for (int k = 1; k < FX_MAXR; ++k) hs.mix((uint64_t)(uint32_t)fx_aff_coef(&a, k));
          hs.mix((uint64_t)(uint32_t)a.tcoef);
          hs.mix((uint64_t)(uint32_t)a.rcoef[0]);
          hs.mix((uint64_t)(uint32_t)a.rcoef[1]);
          if (a.tcoef != 0) {
            if (a.tcoef != 1 || a.base < 0 || (first >= 0 && a.base != first)) { bad = true; return; }
            first = a.base;
          } else {
            hs.mix((uint64_t)(uint32_t)a.base);
          }
        } else {
          if (fx_aff_coef(&a, 0) != 4) { bad = true; return; }
          mix_affine(a);
        }
        if ((x.flags & FX_F_IMM) && which == 2 && x.op == FX_FMUL) var.push_back(x.imm);
        else hs.mix(x.imm);
      } else if (x.op == FX_RBEGIN) {
        // a = loop slot, b = first instruction behind the loop, imm = extent (the class count)
        if (C == 0) C = x.imm;
        if (x.imm != C) { bad = true; return; }
        hs.mix((uint64_t)(uint32_t)x.a);
        hs.mix((uint64_t)(uint32_t)(x.b - (int32_t)pb));
      } else if (x.op == FX_MIFR || x.op == FX_AFFA || x.op == FX_AFFB) {
        if (x.op == FX_MIFR) hs.mix((uint64_t)(uint32_t)(x.a - (int32_t)pb));
        else hs.mix((uint64_t)(uint32_t)x.a);
        mix_affine(aff[x.b]);
        hs.mix(x.imm);
      } else if (x.op == FX_MIF || x.op == FX_MELSE || x.op == FX_RNEXT) {
        hs.mix((uint64_t)(uint32_t)(x.a - (int32_t)pb));
        hs.mix((uint64_t)(uint32_t)x.b);
        hs.mix(x.imm);
      } else {
        hs.mix((uint64_t)(uint32_t)x.a);
        hs.mix((uint64_t)(uint32_t)x.b);
        if (which == 0 && x.op == FX_FGT && (x.flags & FX_F_IMM)) thr_bits = x.imm;            // parameters
        else if (which == 2 && x.op == FX_FMUL && (x.flags & FX_F_IMM)) var.push_back(x.imm);
        else hs.mix(x.imm);
      }
    }
  };
  walk(cl.mask_begin, cl.mask_end, 0);
  hs.mix(cl.mask_vt);
  for (int k = 0; k < 2 && !bad; ++k) {
    hs.mix(outs[k].lead);
    hs.mix(outs[k].pure);
    walk(outs[k].prog_begin, outs[k].prog_end, 1 + k);
  }
  ci.norm_hash = hs.h;
  if (bad || buf_class.size() != 3 || hs.h != kCmapHash) return;
  // the box program multiplies by the size variance, the centre variance, and the same two again
  if (var.size() != 4 || var[0] != var[2] || var[1] != var[3]) return;
  if (C < 2 || C > FX_CMAP_MAX_CLS || first < 0 || (uint32_t)first + cl.n_tasks > C) return;
  ci.conf_slot = (uint32_t)slot_of[0];
  ci.loc_slot = (uint32_t)slot_of[1];
  ci.pri_slot = (uint32_t)slot_of[2];
  ci.C = C;
  ci.first = (uint32_t)first;
  ci.thr_bits = thr_bits;
  ci.var_wh_bits = var[0];
  ci.var_xy_bits = var[1];
  ci.n_rows = cl.n_rows;
  ci.n_tasks = cl.n_tasks;
  for (int k = 0; k < 2; ++k) {
    ci.out_slot[k] = outs[k].ptr_slot;
    ci.out_tstride[k] = outs[k].task_stride;
  }
  ci.ok = true;
}

}  // namespace fx
