// ruy::ThreadPool placeholder. The reference's Context hands out its thread
// pool (ruy/context.h:59-66, ruy/thread_pool.h:61-123); the device path has no
// threads to pool, so this is an empty object kept for source compatibility.
#ifndef RUY_AMD_INCLUDE_RUY_THREAD_POOL_H_
#define RUY_AMD_INCLUDE_RUY_THREAD_POOL_H_

namespace ruy {
class ThreadPool final {};
}  // namespace ruy

#endif  // RUY_AMD_INCLUDE_RUY_THREAD_POOL_H_
