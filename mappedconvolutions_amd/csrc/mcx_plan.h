// Host-side descriptors of map plans (mcx_plan_desc in mcx.h): filled where a plan is built,
// compared with the arguments of every entry point that is handed one.
#pragma once

#include <stdint.h>

#include "mcx.h"
#include "mcx_device.h"

namespace mcx {

constexpr uint32_t kPlanMagic = 0x4d435850u;

// Fold of every field but `check` (FNV-1a over the words): a descriptor that was never filled
// in, or edited afterwards, does not pass.
inline uint64_t plan_desc_fold(const mcx_plan_desc &d) {
  const uint64_t words[] = {d.magic,
                            (uint64_t)(uint32_t)d.kind,
                            (uint64_t)(uint32_t)d.interp,
                            (uint64_t)(uint32_t)d.dtype,
                            (uint64_t)d.SH,
                            (uint64_t)d.SW,
                            (uint64_t)d.MH,
                            (uint64_t)d.MW,
                            (uint64_t)d.K,
                            (uint64_t)d.P,
                            d.plan,
                            d.plan_bytes,
                            d.map,
                            d.iw};
  uint64_t h = 0xcbf29ce484222325ull;
  for (uint64_t w : words)
    for (int i = 0; i < 8; i++) {
      h ^= (w >> (8 * i)) & 0xffu;
      h *= 0x100000001b3ull;
    }
  return h;
}

// SH x SW: the image the map points into; MH x MW: the map.  `dtype`: the type the plan's
// contents depend on (MCX_F32 where they do not).
inline void plan_desc_fill(mcx_plan_desc *d, int kind, int interp, int dtype, int64_t SH,
                           int64_t SW, int64_t MH, int64_t MW, int64_t K, int64_t P,
                           const void *plan, size_t plan_bytes, const void *map, const void *iw) {
  if (!d) return;
  d->magic = kPlanMagic;
  d->kind = kind;
  d->interp = canonical_interp(interp);
  d->dtype = dtype;
  d->SH = SH;
  d->SW = SW;
  d->MH = MH;
  d->MW = MW;
  d->K = K;
  d->P = P;
  d->plan = (uint64_t)(uintptr_t)plan;
  d->plan_bytes = (uint64_t)plan_bytes;
  d->map = (uint64_t)(uintptr_t)map;
  d->iw = (uint64_t)(uintptr_t)iw;
  d->check = plan_desc_fold(*d);
}

// 0 when `d` describes a plan of `kind` for exactly these arguments that lies at `plan`;
// MCX_E_NULL without a descriptor, MCX_E_PLAN on any difference.  `map` / `iw` are compared
// only when check_map (entry points that take the map themselves).
inline int plan_desc_check(const mcx_plan_desc *d, int kind, int interp, int dtype, int64_t SH,
                           int64_t SW, int64_t MH, int64_t MW, int64_t K, int64_t P,
                           const void *plan, size_t plan_bytes, bool check_map, const void *map,
                           const void *iw) {
  if (!d) return MCX_E_NULL;
  if (d->magic != kPlanMagic || d->check != plan_desc_fold(*d)) return MCX_E_PLAN;
  if (d->kind != kind || d->interp != canonical_interp(interp) || d->dtype != dtype)
    return MCX_E_PLAN;
  if (d->SH != SH || d->SW != SW || d->MH != MH || d->MW != MW || d->K != K || d->P != P)
    return MCX_E_PLAN;
  if (d->plan != (uint64_t)(uintptr_t)plan || d->plan_bytes > (uint64_t)plan_bytes)
    return MCX_E_PLAN;
  if (check_map && (d->map != (uint64_t)(uintptr_t)map || d->iw != (uint64_t)(uintptr_t)iw))
    return MCX_E_PLAN;
  return 0;
}

}  // namespace mcx
