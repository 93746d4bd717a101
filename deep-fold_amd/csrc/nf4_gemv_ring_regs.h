// Fixed VGPRs of the ring GEMV kernels (nf4_gemv.hip).  The kernels are compiled with a
// VGPR budget below 128 (amdgpu_num_vgpr), so the compiler never allocates the registers
// named here; they belong to the weight requests in flight and are written and read by asm
// only.  A slot holds one half step: per row an even-aligned pair of dwords of packed bytes
// and one dword of scale.
//   one row per group (RR1): 8 slots          : pairs v104..v119, scales v120..v127
//   gate/up pair      (RR2): 6 slots x 2 rows : pairs v92..v115,  scales v116..v127
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
#define RR2_W_0_0 "v[92:93]"
#define RR2_X_0_0 "v92"
#define RR2_Y_0_0 "v93"
#define RR2_S_0_0 "v116"
#define RR2_CLOB_0_0 "v92", "v93", "v116"
#define RR2_W_0_1 "v[94:95]"
#define RR2_X_0_1 "v94"
#define RR2_Y_0_1 "v95"
#define RR2_S_0_1 "v117"
#define RR2_CLOB_0_1 "v94", "v95", "v117"
#define RR2_W_1_0 "v[96:97]"
#define RR2_X_1_0 "v96"
#define RR2_Y_1_0 "v97"
#define RR2_S_1_0 "v118"
#define RR2_CLOB_1_0 "v96", "v97", "v118"
#define RR2_W_1_1 "v[98:99]"
#define RR2_X_1_1 "v98"
#define RR2_Y_1_1 "v99"
#define RR2_S_1_1 "v119"
#define RR2_CLOB_1_1 "v98", "v99", "v119"
#define RR2_W_2_0 "v[100:101]"
#define RR2_X_2_0 "v100"
#define RR2_Y_2_0 "v101"
#define RR2_S_2_0 "v120"
#define RR2_CLOB_2_0 "v100", "v101", "v120"
#define RR2_W_2_1 "v[102:103]"
#define RR2_X_2_1 "v102"
#define RR2_Y_2_1 "v103"
#define RR2_S_2_1 "v121"
#define RR2_CLOB_2_1 "v102", "v103", "v121"
#define RR2_W_3_0 "v[104:105]"
#define RR2_X_3_0 "v104"
#define RR2_Y_3_0 "v105"
#define RR2_S_3_0 "v122"
#define RR2_CLOB_3_0 "v104", "v105", "v122"
#define RR2_W_3_1 "v[106:107]"
#define RR2_X_3_1 "v106"
#define RR2_Y_3_1 "v107"
#define RR2_S_3_1 "v123"
#define RR2_CLOB_3_1 "v106", "v107", "v123"
#define RR2_W_4_0 "v[108:109]"
#define RR2_X_4_0 "v108"
#define RR2_Y_4_0 "v109"
#define RR2_S_4_0 "v124"
#define RR2_CLOB_4_0 "v108", "v109", "v124"
#define RR2_W_4_1 "v[110:111]"
#define RR2_X_4_1 "v110"
#define RR2_Y_4_1 "v111"
#define RR2_S_4_1 "v125"
#define RR2_CLOB_4_1 "v110", "v111", "v125"
#define RR2_W_5_0 "v[112:113]"
#define RR2_X_5_0 "v112"
#define RR2_Y_5_0 "v113"
#define RR2_S_5_0 "v126"
#define RR2_CLOB_5_0 "v112", "v113", "v126"
#define RR2_W_5_1 "v[114:115]"
#define RR2_X_5_1 "v114"
#define RR2_Y_5_1 "v115"
#define RR2_S_5_1 "v127"
#define RR2_CLOB_5_1 "v114", "v115", "v127"

// The pair ring has six slots; the names of slots 6 and 7 exist only so that code shared with
// the eight-slot ring still parses in branches that are compiled out.
#define RR2_W_6_0 RR2_W_0_0
#define RR2_X_6_0 RR2_X_0_0
#define RR2_Y_6_0 RR2_Y_0_0
#define RR2_S_6_0 RR2_S_0_0
#define RR2_CLOB_6_0 RR2_CLOB_0_0
#define RR2_W_6_1 RR2_W_0_1
#define RR2_X_6_1 RR2_X_0_1
#define RR2_Y_6_1 RR2_Y_0_1
#define RR2_S_6_1 RR2_S_0_1
#define RR2_CLOB_6_1 RR2_CLOB_0_1
#define RR2_W_7_0 RR2_W_0_0
#define RR2_X_7_0 RR2_X_0_0
#define RR2_Y_7_0 RR2_Y_0_0
#define RR2_S_7_0 RR2_S_0_0
#define RR2_CLOB_7_0 RR2_CLOB_0_0
#define RR2_W_7_1 RR2_W_0_1
#define RR2_X_7_1 RR2_X_0_1
#define RR2_Y_7_1 RR2_Y_0_1
#define RR2_S_7_1 RR2_S_0_1
#define RR2_CLOB_7_1 RR2_CLOB_0_1

#define RR1_W(q) RR1_W_##q
#define RR1_X(q) RR1_X_##q
#define RR1_Y(q) RR1_Y_##q
#define RR1_S(q) RR1_S_##q
#define RR1_CLOB(q) RR1_CLOB_##q
#define RR2_W(q, r) RR2_W_##q##_##r
#define RR2_X(q, r) RR2_X_##q##_##r
#define RR2_Y(q, r) RR2_Y_##q##_##r
#define RR2_S(q, r) RR2_S_##q##_##r
#define RR2_CLOB(q, r) RR2_CLOB_##q##_##r
