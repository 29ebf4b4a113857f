// Compiler-builtin spellings so that the sources need no HIP header (they are
// compiled by hiprtc at model-compile time and by plain hipcc in checks).
#define DNX_INLINE inline __attribute__((always_inline))
#define DNX_TID ((int)__builtin_amdgcn_workitem_id_x())
#define DNX_BID_X ((unsigned)__builtin_amdgcn_workgroup_id_x())
#define DNX_BID_Y ((unsigned)__builtin_amdgcn_workgroup_id_y())
#define DNX_BID_Z ((unsigned)__builtin_amdgcn_workgroup_id_z())
typedef __SIZE_TYPE__ size_t;
#define DNX_LAUNCH_BOUNDS(n) __attribute__((amdgpu_flat_work_group_size(1, n)))
// workgroup barrier with LDS/global visibility, what __syncthreads() expands to
#define DNX_SYNC()                                                             \
  do {                                                                         \
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");                     \
    __builtin_amdgcn_s_barrier();                                              \
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");                     \
  } while (0)
