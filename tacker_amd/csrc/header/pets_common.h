// Device-wide constants shared by every kernel header.
// Replaces src/header/pets_common.h of the reference: SM_NUM (142, a compile-time
// macro there) becomes the MI355X compute-unit count, which the host also
// queries at run time (tkGetCuCount); the int8 experiment switch is gone.
#pragma once
#define TK_WAVE_SIZE 64
#define TK_CU_NUM 256       // MI355X: 8 XCDs x 32 CUs
#define TK_XCD_NUM 8
