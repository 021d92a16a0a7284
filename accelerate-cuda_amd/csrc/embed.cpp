// The device headers travel inside the library: they are pasted into the
// object file by the assembler and handed to hiprtc by name at compile time,
// so an installed libacchip.so needs no side files.
#include <cstring>

#include "acc_internal.hpp"

#define ACC_EMBED(sym, file)                                        \
  __asm__(".section .rodata\n"                                      \
          ".global acc_embed_" #sym "_begin\n"                      \
          "acc_embed_" #sym "_begin:\n"                             \
          ".incbin \"" file "\"\n"                                  \
          ".global acc_embed_" #sym "_end\n"                        \
          "acc_embed_" #sym "_end:\n"                               \
          ".byte 0\n"                                               \
          ".previous\n");                                           \
  extern "C" const char acc_embed_##sym##_begin[];                  \
  extern "C" const char acc_embed_##sym##_end[];

ACC_EMBED(device, "device/acc_hip_device.h")
ACC_EMBED(prim, "device/acc_prim.h")
ACC_EMBED(map, "device/skel_map.h")
ACC_EMBED(fold, "device/skel_fold.h")
ACC_EMBED(foldseg, "device/skel_foldseg.h")
ACC_EMBED(scan, "device/skel_scan.h")
ACC_EMBED(permute, "device/skel_permute.h")
ACC_EMBED(stencil, "device/skel_stencil.h")
ACC_EMBED(stencil_nd, "device/skel_stencil_nd.h")

namespace acc {

const std::vector<EmbeddedHeader> &embedded_headers()
{
  static const std::vector<EmbeddedHeader> headers = {
      {"acc_hip_device.h", acc_embed_device_begin, acc_embed_device_end},
      {"acc_prim.h", acc_embed_prim_begin, acc_embed_prim_end},
      {"skel_map.h", acc_embed_map_begin, acc_embed_map_end},
      {"skel_fold.h", acc_embed_fold_begin, acc_embed_fold_end},
      {"skel_foldseg.h", acc_embed_foldseg_begin, acc_embed_foldseg_end},
      {"skel_scan.h", acc_embed_scan_begin, acc_embed_scan_end},
      {"skel_permute.h", acc_embed_permute_begin, acc_embed_permute_end},
      {"skel_stencil.h", acc_embed_stencil_begin, acc_embed_stencil_end},
      {"skel_stencil_nd.h", acc_embed_stencil_nd_begin, acc_embed_stencil_nd_end},
  };
  return headers;
}

std::string embedded_text(const char *name)
{
  for (const EmbeddedHeader &h : embedded_headers())
    if (std::strcmp(h.name, name) == 0) return std::string(h.begin, h.end);
  return std::string();
}

}  // namespace acc
