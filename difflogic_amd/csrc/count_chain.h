// Geometry of the chained count kernel (dl_logic_eval_chained_groupbitsum), shared by the kernel
// and the host-side plan builder.
#pragma once

#define DL_CC_WAVES 16                                  // waves per workgroup (one workgroup per CU)
#define DL_CC_WAVE_STEPS 8                              // steps a wave walks per block
#define DL_CC_MAX_BLOCKS 16                             // blocks per workgroup: 16, 8, 4, 2 or 1 (chosen by the plan)
#define DL_CC_BLOCK (DL_CC_WAVES * DL_CC_WAVE_STEPS)    // outputs parked in LDS per block
#define DL_CC_MAX_WG_STEPS (DL_CC_BLOCK * DL_CC_MAX_BLOCKS)   // schedules are padded to whole multiples of this
#define DL_CC_MAX_CLASSES (2 * DL_CC_WAVES)             // a wave owns at most two classes
#define DL_CC_PLANES 8                                  // counter planes per class and workgroup: counts up to 255
