/*
 * Stream<gpu> and the error glue between the C ABI and mshadow's CHECK convention.
 *
 * Stream<gpu> keeps the members callers touch in the reference
 * (mshadow/stream_gpu-inl.h:18-180): stream_, dev_id, Wait(), CheckIdle(),
 * GetStream(); the BLAS / solver / DNN handle members exist but are inert: the library
 * behind the C ABI keeps its own rocBLAS handle per thread and device and binds it to the
 * stream of each call, and there is no solver or DNN engine. A NULL stream is fatal when MSHADOW_FORCE_STREAM
 * is on, and otherwise means the device's default stream (:79-88).
 */
#ifndef MSHADOW_HIP_STREAM_H_
#define MSHADOW_HIP_STREAM_H_

#include <mshadow_hip.h>

#include <string>

#include "../core/tensor_types.h"

/*! \brief turn a non-zero ABI status into mshadow's fatal error. A failure reported
 *  while the runtime is unloading is thrown instead of aborting, so that destructors
 *  running at process exit can swallow it (mshadow/base.h:252-276). */
#define MSHADOW_HIP_CALL(func)                                                  \
  {                                                                             \
    int e_ = (func);                                                            \
    if (e_ != MSHADOW_HIP_OK) {                                                 \
      std::string msg_ = mshadow_hip_last_error();                              \
      if (msg_.find("unload") != std::string::npos ||                           \
          msg_.find("shutting down") != std::string::npos ||                    \
          msg_.find("deinitialized") != std::string::npos) {                    \
        throw dmlc::Error(msg_);                                                \
      }                                                                         \
      LOG(FATAL) << "HIP: " << msg_;                                            \
    }                                                                           \
  }
/*! \brief run func, ignoring the error class that MSHADOW_HIP_CALL throws */
#define MSHADOW_CATCH_ERROR(func)                                               \
  {                                                                             \
    try {                                                                       \
      (func);                                                                   \
    } catch (const dmlc::Error &e) {                                            \
      std::string what = e.what();                                              \
      if (what.find("shutting down") == std::string::npos &&                    \
          what.find("unload") == std::string::npos) {                           \
        LOG(ERROR) << "Ignore HIP Error " << what;                              \
      }                                                                         \
    }                                                                           \
  }

namespace mshadow {

template <>
struct Stream<gpu> {
  /*! \brief handle ownership states, kept for source compatibility */
  enum HandleState { NoHandle = 0, OwnHandle = 1 };
  /*! \brief opaque stream handle of the C ABI (a hipStream_t underneath) */
  void *stream_;
  HandleState blas_handle_ownership_;
  HandleState solver_handle_ownership_;
  HandleState dnn_handle_ownership_;
  /*! \brief properties of device dev_id, filled by NewStream when dev_id != -1 */
  mshadow_hip_props prop;
  /*! \brief device the stream was created for, -1 if unspecified */
  int dev_id;

  Stream(void)
      : stream_(NULL), blas_handle_ownership_(NoHandle), solver_handle_ownership_(NoHandle),
        dnn_handle_ownership_(NoHandle), dev_id(-1) {}
  /*! \brief block the host until everything queued on this stream has finished */
  inline void Wait(void) { MSHADOW_HIP_CALL(mshadow_hip_stream_sync(stream_)); }
  /*! \brief true if nothing queued on this stream is still running */
  inline bool CheckIdle(void) {
    int idle = 0;
    MSHADOW_HIP_CALL(mshadow_hip_stream_query(stream_, &idle));
    return idle != 0;
  }
  /*! \brief the raw handle to pass to the C ABI */
  inline static void *GetStream(Stream<gpu> *stream) {
    if (stream == NULL) {
#if MSHADOW_FORCE_STREAM
      LOG(FATAL) << "Default GPU stream was used when MSHADOW_FORCE_STREAM was on";
#endif
      return NULL;
    }
    return stream->stream_;
  }
  /* handles are owned by the library (BLAS) or do not exist (solver, DNN): creation is
     accepted and ignored */
  inline void CreateBlasHandle() {}
  inline void DestroyBlasHandle() {}
  inline void CreateSolverHandle() {}
  inline void DestroySolverHandle() {}
  inline void CreateDnnHandle() {}
  inline void DestroyDnnHandle() {}
};

template <>
inline void DeleteStream<gpu>(Stream<gpu> *stream) {
  if (stream == NULL) return;
  MSHADOW_HIP_CALL(mshadow_hip_stream_destroy(stream->stream_));
  delete stream;
}

template <>
inline Stream<gpu> *NewStream<gpu>(bool create_blas_handle, bool create_dnn_handle, int dev_id) {
  Stream<gpu> *st = new Stream<gpu>();
  int e = mshadow_hip_stream_create(&st->stream_);
  if (e != MSHADOW_HIP_OK) {
    delete st;
    LOG(FATAL) << "HIP: " << mshadow_hip_last_error();
  }
  st->dev_id = dev_id;
  if (dev_id != -1) {
    MSHADOW_HIP_CALL(mshadow_hip_get_props(dev_id, &st->prop));
  }
  return st;
}

}  // namespace mshadow
#endif  // MSHADOW_HIP_STREAM_H_
