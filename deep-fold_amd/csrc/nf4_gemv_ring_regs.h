// Fixed VGPRs of the ring GEMV kernels (nf4_gemv.hip).  The kernels are compiled with a
// VGPR budget below 128 (amdgpu_num_vgpr), so the compiler never allocates the registers
// named here; they belong to the weight requests in flight and are written and read by asm
// only.  A slot holds one half step: per row an even-aligned pair of dwords of packed bytes
// and one dword of scale: 8 slots, pairs v104..v119, scales v120..v127.
#pragma once

#define RR1_W_0 "v[104:105]"
#define RR1_X_0 "v104"
#define RR1_Y_0 "v105"
#define RR1_S_0 "v120"
#define RR1_CLOB_0 "v104", "v105", "v120"
#define RR1_W_1 "v[106:107]"
#define RR1_X_1 "v106"
#define RR1_Y_1 "v107"
#define RR1_S_1 "v121"
#define RR1_CLOB_1 "v106", "v107", "v121"
#define RR1_W_2 "v[108:109]"
#define RR1_X_2 "v108"
#define RR1_Y_2 "v109"
#define RR1_S_2 "v122"
#define RR1_CLOB_2 "v108", "v109", "v122"
#define RR1_W_3 "v[110:111]"
#define RR1_X_3 "v110"
#define RR1_Y_3 "v111"
#define RR1_S_3 "v123"
#define RR1_CLOB_3 "v110", "v111", "v123"
#define RR1_W_4 "v[112:113]"
#define RR1_X_4 "v112"
#define RR1_Y_4 "v113"
#define RR1_S_4 "v124"
#define RR1_CLOB_4 "v112", "v113", "v124"
#define RR1_W_5 "v[114:115]"
#define RR1_X_5 "v114"
#define RR1_Y_5 "v115"
#define RR1_S_5 "v125"
#define RR1_CLOB_5 "v114", "v115", "v125"
#define RR1_W_6 "v[116:117]"
#define RR1_X_6 "v116"
#define RR1_Y_6 "v117"
#define RR1_S_6 "v126"
#define RR1_CLOB_6 "v116", "v117", "v126"
#define RR1_W_7 "v[118:119]"
#define RR1_X_7 "v118"
#define RR1_Y_7 "v119"
#define RR1_S_7 "v127"
#define RR1_CLOB_7 "v118", "v119", "v127"

// The pair ring has six slots; the names of slots 6 and 7 exist only so that code shared with
// the eight-slot ring still parses in branches that are compiled out.

#define RR1_W(q) RR1_W_##q
#define RR1_X(q) RR1_X_##q
#define RR1_Y(q) RR1_Y_##q
#define RR1_S(q) RR1_S_##q
#define RR1_CLOB(q) RR1_CLOB_##q
