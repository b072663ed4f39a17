// Device-side building blocks shared by every run-time compiled kernel (placed after thorhip_numeric.h).
#pragma once
