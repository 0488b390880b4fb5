/*
 * FlagCX ABI constants and opaque handle types used at the drop-in boundary.
 * The numeric values are the ABI of flagcx/include/flagcx.h (result codes
 * :21-33, data types :36-53, reduction ops :57-66, memcpy / memory / event
 * kinds :87-102) and must not change.  A translation unit that already
 * includes the real flagcx.h gets the same names from there.
 */
#ifndef FLAGCX_AMD_FX_TYPES_H_
#define FLAGCX_AMD_FX_TYPES_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#ifndef FLAGCX_H_ /* the real flagcx.h was not included */

typedef enum {
  flagcxSuccess = 0,              flagcxUnhandledDeviceError = 1,
  flagcxSystemError = 2,          flagcxInternalError = 3,
  flagcxInvalidArgument = 4,      flagcxInvalidUsage = 5,
  flagcxRemoteError = 6,          flagcxInProgress = 7,
  flagcxUnhandledCCLError = 8,    flagcxNotSupported = 9,
  flagcxNumResults = 10
} flagcxResult_t;

typedef enum {
  flagcxInt8 = 0,    flagcxChar = 0,    flagcxUint8 = 1,
  flagcxInt32 = 2,   flagcxInt = 2,     flagcxUint32 = 3,
  flagcxInt64 = 4,   flagcxUint64 = 5,
  flagcxFloat16 = 6, flagcxHalf = 6,
  flagcxFloat32 = 7, flagcxFloat = 7,
  flagcxFloat64 = 8, flagcxDouble = 8,
  flagcxBfloat16 = 9, flagcxNumTypes = 10
} flagcxDataType_t;

typedef enum {
  flagcxSum = 0, flagcxProd = 1, flagcxMax = 2, flagcxMin = 3, flagcxAvg = 4,
  flagcxRedNoOp = 5, flagcxNumRedOps = 5, flagcxMaxRedOp = 0x7fffffff
} flagcxRedOp_t;

typedef enum {
  flagcxMemcpyHostToDevice = 0,
  flagcxMemcpyDeviceToHost = 1,
  flagcxMemcpyDeviceToDevice = 2
} flagcxMemcpyType_t;

typedef enum {
  flagcxMemHost = 0, /* pinned */
  flagcxMemDevice = 1,
  flagcxMemManaged = 2
} flagcxMemType_t;

typedef enum {
  flagcxEventDefault = 0,
  flagcxEventDisableTiming = 1
} flagcxEventType_t;

/* flagcx/include/flagcx.h:112-116 */
#define FLAGCX_UNIQUE_ID_BYTES 256
typedef struct {
  char internal[FLAGCX_UNIQUE_ID_BYTES];
} flagcxUniqueId;
typedef flagcxUniqueId *flagcxUniqueId_t;

typedef struct flagcxComm *flagcxComm_t;
typedef struct flagcxStream *flagcxStream_t;
typedef struct flagcxEvent *flagcxEvent_t;
typedef struct flagcxIpcMemHandle *flagcxIpcMemHandle_t;

#endif /* FLAGCX_H_ */

#ifdef __cplusplus
}
#endif
#endif /* FLAGCX_AMD_FX_TYPES_H_ */
