// Element dtype ids shared by host and device code (same values as MTQ_F32 /
// MTQ_F16 / MTQ_BF16 of the public header).
#pragma once
namespace mtq {
enum : int { DT_F32 = 0, DT_F16 = 1, DT_BF16 = 2 };
}
