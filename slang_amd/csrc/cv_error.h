// cv_error.h -- per-thread error message shared by the translation units that export C entry points.
#pragma once
#include "../../include/coopvec.h"

namespace cv {
// Records a printf-style message for cvGetLastErrorMessage() on the calling thread; returns `code`.
CvResult failWith(CvResult code, const char* fmt, ...);
// Records (printf-style) which kernel a launcher dispatched, for cvGetLastKernelName() on the calling
// thread.  `append` adds to the current name (" + second kernel") instead of replacing it.
void noteKernel(bool append, const char* fmt, ...);
}
