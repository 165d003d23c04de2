/* Shared between the translation units of liblutgemm_gfx950.so; not installed. */
#ifndef LUTGEMM_INTERNAL_H
#define LUTGEMM_INTERNAL_H

/* Records a HIP error for lutgemm_last_hip_error() on this thread and returns
 * LUTGEMM_EHIP. */
int lutgemm_internal_hip_fail(int hip_error);

#endif
