// The kernels of the embedded code objects: for each (module, name) the argument signature the launch checks, the
// -D names that select a compiled variant, and the -D names whose values ride along as trailing int arguments.
// Signature letters: p = device buffer (8 bytes), i = int / uint (4), f = float (4), z = size_t by value (8).
#pragma once

struct HiddenDef {
  const char* name;  // nullptr ends the list; "LDS" is not an argument: it is the launch's dynamic LDS size in bytes;
                     // "SOFTCAP" and "RSCALE" are read as floats ("-DSOFTCAP=30.0f") and ride along as their bit patterns
  int def;
  bool required;
};
struct KernelSpec {
  const char* which;
  const char* name;
  const char* requires_def;  // this entry is taken only when the -D string holds this name (nullptr: always)
  const char* args;
  const char* variant[8];  // nullptr-terminated
  HiddenDef hidden[6];     // {nullptr} terminated
  int local_x;             // threads per work-group the kernel is written for (0 = any)
};

// Entries with requires_def come before the plain entry of the same name.
static const KernelSpec kKernelTable[] = {
    // ---- ops (Q2_AQ / Q2_SC / Q2_AB: the two-pass mode's residual offsets, the reference's -D names; 0 = one pass)
    {"ops", "quant_rows", nullptr, "piiiipppi", {nullptr}, {{"Q2_AQ", 0, false}, {"Q2_SC", 0, false}, {"Q2_AB", 0, false}, {nullptr, 0, false}}, 256},
    {"ops", "rmsnorm_quant", nullptr, "pipiiifppppii", {nullptr}, {{"Q2_AQ", 0, false}, {"Q2_SC", 0, false}, {"Q2_AB", 0, false}, {nullptr, 0, false}}, 256},
    {"ops", "swiglu_quant", nullptr, "piiipppiii", {nullptr}, {{"Q2_AQ", 0, false}, {"Q2_SC", 0, false}, {"Q2_AB", 0, false}, {nullptr, 0, false}}, 256},
    {"ops", "rmsnorm_quant_r16", nullptr, "pipiiifppppii", {nullptr}, {{nullptr, 0, false}}, 256},
    {"ops", "swiglu_quant_r16", nullptr, "piiipppiii", {nullptr}, {{nullptr, 0, false}}, 256},
    {"ops", "add_norm_quant", nullptr, "pppiffpiipppii", {nullptr}, {{"Q2_AQ", 0, false}, {"Q2_SC", 0, false}, {"Q2_AB", 0, false}, {nullptr, 0, false}}, 256},
    {"ops", "act_usum", nullptr, "ppip", {nullptr}, {{nullptr, 0, false}}, 256},
    {"ops", "q4k_wscales", nullptr, "pziip", {nullptr}, {{nullptr, 0, false}}, 256},
    {"ops", "act_usum_bf16", nullptr, "ppip", {nullptr}, {{nullptr, 0, false}}, 256},
    {"ops", "q4k_wscales_bf16", nullptr, "pziip", {nullptr}, {{nullptr, 0, false}}, 256},
    {"ops", "q4k_wscales_int", nullptr, "pziip", {nullptr}, {{nullptr, 0, false}}, 256},
    {"ops", "asc_expand", nullptr, "ppii", {nullptr}, {{nullptr, 0, false}}, 256},
    {"ops", "softcap_rows", nullptr, "piiif", {nullptr}, {{nullptr, 0, false}}, 0},
    {"ops", "fill32", nullptr, "piz", {nullptr}, {{nullptr, 0, false}}, 256},
    {"ops", "copy128", nullptr, "ppz", {nullptr}, {{nullptr, 0, false}}, 256},
    {"ops", "read_probe", nullptr, "pzp", {nullptr}, {{nullptr, 0, false}}, 256},
    {"ops", "mfma_probe", nullptr, "pi", {nullptr}, {{nullptr, 0, false}}, 256},
    // ---- decode
    // (-DSCHED=n: the LDS-staged GEMVs' row schedule for the launch's grid, worked out by the launcher -- see
    //  gemv_lds.inc; left out, the kernel works it out itself)
    {"decode", "gemv", "GU2", "piippppipiip", {"QT", "LPR", "PF", "GU2", nullptr}, {{"LDS", 0, true}, {"SCHED", -1, false}, {nullptr, 0, false}}, 256},
    {"decode", "gemv", "BT", "piippppipii", {"QT", "LPR", "PF", "BT", nullptr},
     {{"LDS", 0, true}, {"SOFTCAP", 0, false}, {"SCHED", -1, false}, {nullptr, 0, false}}, 512},
    {"decode", "gemv_mt", "BT", "piippppiipiii", {"QT", "LPR", "PF", "TB", "BT", nullptr},
     {{"LDS", 0, true}, {"Q2_AQ", 0, false}, {"Q2_SC", 0, false}, {"SOFTCAP", 0, false}, {"SCHED", -1, false}, {nullptr, 0, false}}, 512},
    {"decode", "gemv", nullptr, "piippppipii", {"QT", "LPR", "PF", nullptr},
     {{"LDS", 0, true}, {"SOFTCAP", 0, false}, {"SCHED", -1, false}, {nullptr, 0, false}}, 256},
    {"decode", "gemv_mt", nullptr, "piippppiipiii", {"QT", "LPR", "PF", "TB", nullptr},
     {{"LDS", 0, true}, {"Q2_AQ", 0, false}, {"Q2_SC", 0, false}, {"SOFTCAP", 0, false}, {"SCHED", -1, false}, {nullptr, 0, false}}, 256},
    {"decode", "gemv_mm_reduce", nullptr, "pipiiiii", {nullptr}, {{nullptr, 0, false}}, 256},
    {"decode", "gemv_mm", nullptr, "piippppiipiiiii", {"QT", nullptr}, {{nullptr, 0, false}}, 512},
    {"decode", "moe_gateup_q", "ROUTE", "ppiipppippppipppppppiiipp", {"QT", "GROWS", "TM", "QUANT", "ROUTE", nullptr}, {{"NE", 0, true}, {nullptr, 0, false}}, 512},
    {"decode", "moe_gateup_q", "QUANT", "ppiipppippppippp", {"QT", "GROWS", "TM", "QUANT", nullptr}, {{"NE", 0, true}, {nullptr, 0, false}}, 512},
    {"decode", "moe_down1_q", nullptr, "piipppipppppi", {"QT", "GROWS", nullptr}, {{"NE", 0, true}, {nullptr, 0, false}}, 256},
    {"decode", "moe_gateup_q", nullptr, "ppiipppipppp", {"QT", "GROWS", "TM", nullptr}, {{"NE", 0, true}, {nullptr, 0, false}}, 256},
    {"decode", "moe_down_q", nullptr, "piipppipppp", {"QT", "GROWS", "TM", nullptr}, {{"NE", 0, true}, {nullptr, 0, false}}, 256},
    {"decode", "expand_iq3s", nullptr, "pppii", {nullptr}, {{nullptr, 0, false}}, 256},
    {"decode", "expand_q3k", nullptr, "ppii", {nullptr}, {{nullptr, 0, false}}, 256},
    {"decode", "expand_iq3xxs", nullptr, "pppii", {nullptr}, {{nullptr, 0, false}}, 256},
    {"decode", "gemv_v", nullptr, "piippppipii", {"QT", "GROWS", nullptr}, {{"SOFTCAP", 0, false}, {nullptr, 0, false}}, 256},
    {"decode", "gemv_mt_v", nullptr, "piippppiipiii", {"QT", "GROWS", "TB", nullptr}, {{"SOFTCAP", 0, false}, {nullptr, 0, false}}, 256},
    // ---- gemm
    // (-DHDT / -DHDS / -DHD = 1 or 2: the Q6_K kernels on planes written out from IQ3_XXS or IQ3_S)
    // (-DPRE=1: the Q4_K tile kernels with the scale vectors ready-made, two more buffers behind the plain form's)
    {"gemm", "gemm", "PRE", "ppppppiiiiippiipipipp", {"QTYPE", "ACT32", "MOE_TILES", "PRE", nullptr},
     {{"NE", 0, true}, {nullptr, 0, false}}, 256},
    {"gemm", "gemm", "PRE64", "ppppppiiiiiiiii", {"QTYPE", "ACT32", "BM", "BN", "PRE64", nullptr}, {{nullptr, 0, false}}, 256},
    {"gemm", "gemm", "HDT", "ppppppiiiiippiipipi", {"QTYPE", "ACT32", "MOE_TILES", "HDT", nullptr},
     {{"NE", 0, true}, {nullptr, 0, false}}, 256},
    {"gemm", "gemm", "HDS", "ppppppiiiiiiiii", {"QTYPE", "ACT32", "BM", "BN", "SPLITK", "HDS", nullptr}, {{nullptr, 0, false}}, 256},
    {"gemm", "gemm", "HD", "ppppppiiiiiiiii", {"QTYPE", "ACT32", "HD", nullptr}, {{nullptr, 0, false}}, 256},
    {"gemm", "gemm", "MOE_TILES", "ppppppiiiiippiipipi", {"QTYPE", "ACT32", "MOE_TILES", nullptr},
     {{"NE", 0, true}, {nullptr, 0, false}}, 256},
    {"gemm", "gemm", "SPLITK", "ppppppiiiiiiiii", {"QTYPE", "ACT32", "BM", "BN", "SPLITK", nullptr}, {{nullptr, 0, false}}, 256},
    {"gemm", "gemm", "BN", "ppppppiiiiiiiii", {"QTYPE", "ACT32", "BM", "BN", nullptr}, {{nullptr, 0, false}}, 256},
    {"gemm", "gemm", "WM", "ppppppiiiiiiiii", {"QTYPE", "ACT32", "AU", "WM", nullptr}, {{nullptr, 0, false}}, 512},
    {"gemm", "gemm", "AU", "ppppppiiiiiiiii", {"QTYPE", "ACT32", "AU", nullptr}, {{nullptr, 0, false}}, 256},
    {"gemm", "gemm", "BM", "ppppppiiiiiiiii", {"QTYPE", "ACT32", "BM", nullptr}, {{nullptr, 0, false}}, 256},
    {"gemm", "gemm", nullptr, "ppppppiiiiiiiii", {"QTYPE", "ACT32", nullptr}, {{nullptr, 0, false}}, 256},
    {"gemm", "gemm_simple", "MOE_TILES", "ppppppiiiiippiipipi", {"QTYPE", "ACT32", "MOE_TILES", nullptr},
     {{"NE", 0, true}, {nullptr, 0, false}}, 256},
    {"gemm", "gemm_simple", nullptr, "ppppppiiiiiiiii", {"QTYPE", "ACT32", nullptr}, {{nullptr, 0, false}}, 256},
    {"gemm", "splitk_reduce", nullptr, "pipiiiii", {nullptr}, {{nullptr, 0, false}}, 256},
    {"gemm", "moe_gateup_q", "PRE", "ppiipppippppippppppp", {"QT", "QUANT", "PRE", nullptr}, {{"NE", 0, true}, {nullptr, 0, false}}, 256},
    {"gemm", "moe_gateup_q", "QUANT", "ppiipppippppippp", {"QT", "QUANT", nullptr}, {{"NE", 0, true}, {nullptr, 0, false}}, 256},
    {"gemm", "moe_gateup_q", nullptr, "ppiipppipppp", {"QT", nullptr}, {{"NE", 0, true}, {nullptr, 0, false}}, 256},
    // ---- moe
    {"moe", "moe_route", "USUM", "piippppppipi", {"USUM", nullptr}, {{"NE", 0, true}, {"NU", 0, true}, {"NPART", 1, false}, {nullptr, 0, false}}, 256},
    {"moe", "moe_route", "ESCALE", "piippppp", {"ESCALE", nullptr}, {{"NE", 0, true}, {"NU", 0, true}, {"NPART", 1, false}, {nullptr, 0, false}}, 256},
    {"moe", "moe_route", "ROUTE_DS", "piippppp", {"ROUTE_DS", nullptr},
     {{"NE", 0, true}, {"NU", 0, true}, {"NPART", 1, false}, {"RSCALE", 0x3F800000, false}, {nullptr, 0, false}}, 256},
    {"moe", "moe_route1", "ESCALE", "ppppppp", {"ESCALE", nullptr},
     {{"NE", 0, true}, {"NU", 0, true}, {"HAS_GATE", 0, false}, {nullptr, 0, false}}, 64},
    {"moe", "moe_route1", "ROUTE_DS", "ppppppp", {"ROUTE_DS", nullptr},
     {{"NE", 0, true}, {"NU", 0, true}, {"HAS_GATE", 0, false}, {"RSCALE", 0x3F800000, false}, {nullptr, 0, false}}, 64},
    {"moe", "moe_route", nullptr, "piipppp", {nullptr}, {{"NE", 0, true}, {"NU", 0, true}, {"NPART", 1, false}, {nullptr, 0, false}}, 256},
    {"moe", "moe_route1", nullptr, "pppppp", {nullptr},
     {{"NE", 0, true}, {"NU", 0, true}, {"HAS_GATE", 0, false}, {nullptr, 0, false}}, 64},
    {"moe", "moe_route_small", nullptr, "piippppppp", {nullptr},
     {{"NE", 0, true}, {"NU", 0, true}, {"TM", 16, false}, {nullptr, 0, false}}, 512},
    {"moe", "moe_scan", nullptr, "ppppp", {nullptr}, {{"NE", 0, true}, {"TM", 16, false}, {"NCH", 1, false}, {nullptr, 0, false}}, 1024},
    {"moe", "moe_scatter", nullptr, "ppipppp", {nullptr}, {{"NU", 0, true}, {"NE", 0, true}, {"NPART", 0, true}, {nullptr, 0, false}}, 512},
    {"moe", "moe_quant", nullptr, "piipp", {nullptr}, {{"FV", 1 << 30, false}, {nullptr, 0, false}}, 256},
    {"moe", "moe_quant_sums", nullptr, "piippp", {nullptr}, {{"FV", 1 << 30, false}, {nullptr, 0, false}}, 256},
    {"moe", "moe_combine", nullptr, "pppppi", {nullptr}, {{"NU", 0, true}, {nullptr, 0, false}}, 256},
};
