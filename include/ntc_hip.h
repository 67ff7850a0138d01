/*
 * ntc_hip.h - C ABI of the MI355X (gfx950) neural-texture-set decoder.
 *
 * This is the seam a LibNTC maintainer binds in place of the CUDA launchers that
 * ITextureSet::Decompress drives (reference src/TextureSet.cpp:1664-1897):
 *
 *   reference call (file:line)                                replaced by
 *   --------------------------------------------------------  -------------------------
 *   cuda::Inference(InferenceKernelParams const&)             ntc_hip_decode (one launch for
 *     src/Regression.h:37, src/Inference.cu:159-165            every mip of every set)
 *   cuda::UnpackLatents  src/Quantizer.h:56-62                 fused into ntc_hip_decode
 *   cuda::ConvertNetworkFromQuantizedToFp16                    deleted: the int8 blob of
 *     src/Quantizer.h:35-40                                    src/WeightLayout.cpp:142-268
 *                                                              is consumed as stored
 *   cuda::CopyImage (1:1 branch) src/ImageProcessing.h:76-80   fused output formats below
 *   cudaMalloc / cudaMemcpy / cudaEvent* used by that path     ntc_hip_alloc / upload / ...
 *
 * Plain C: pointers, sizes and PODs only.  Every entry point returns 0 on success,
 * a positive hipError_t value when a HIP call failed, or a negative NtcHipError.
 * A message for the last failure on the calling thread is kept per thread, like
 * the reference's thread-local error buffer (src/Errors.cpp:21-52).
 *
 * Contexts: all device state - the device, a stream, the decode kernels' mip table with its staging
 * memory, the loss pass's partial sums, timing events - belongs to an NtcHipContext (ntc_hip_create /
 * ntc_hip_destroy), as the reference scopes its device per context (include/libntc/ntc.h:1289-1290,
 * src/CudaDeviceGuard.cpp:21-62).  Every entry point exists as ntc_hip_ctx_<name>(context, ...); the
 * functions without a context argument run on one default context that ntc_hip_init creates.  Contexts
 * share nothing (except the per-device table of ntc_hip_decode_static, see there); each queues its work
 * on its own stream in call order, and ntc_hip_ctx_synchronize waits for it.  A call makes its context's
 * device current and restores the caller's before it returns.
 * Threading: the reference has no locks (its texture sets share __constant__ state,
 * src/Regression.cu:40-51); here only the list of live contexts is guarded.  Calls on ONE context must be
 * serialised by the caller; different contexts may be used from different threads at the same time -
 * with ONE exception: ntc_hip_decode_static, whose table is one array per GPU shared by every context on it,
 * so its calls must be serialised per GPU, across contexts (see there).  A destroyed context's handle is
 * refused by every entry point (NTC_HIP_ERR_NOT_INITIALIZED) until a later ntc_hip_create happens to return
 * the same address.
 */
#ifndef NTC_HIP_H
#define NTC_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NTC_HIP_MAX_MIPS      16 /* NTC_MAX_MIPS,     include/libntc/shaders/InferenceConstants.h:22 */
#define NTC_HIP_MAX_CHANNELS  16 /* NTC_MAX_CHANNELS, include/libntc/shaders/InferenceConstants.h:23 */
#define NTC_HIP_MLP_LAYERS    4  /* NTC_MLP_LAYERS,   include/libntc/shaders/InferenceConstants.h:28 */
#define NTC_HIP_MAX_LAYER_WIDTH 64

typedef enum NtcHipError {
    NTC_HIP_OK                 = 0,
    NTC_HIP_ERR_INVALID_ARG    = -1,
    NTC_HIP_ERR_UNSUPPORTED    = -2, /* a decoder spec no compiled kernel covers */
    NTC_HIP_ERR_NO_DEVICE      = -3,
    NTC_HIP_ERR_NOT_INITIALIZED= -4
} NtcHipError;

/* How one latent grid feeds the network input vector. */
typedef enum NtcHipGridMode {
    /* 4-tap bilinear filter with wrap addressing, one input per feature
     * (src/FeatureGridDevice.h:33-98, include/libntc/shaders/Inference.hlsli:62-87). */
    NTC_HIP_GRID_BILINEAR  = 0,
    /* The four unfiltered neighbours a00,a01,a10,a11 of src/FeatureGridDevice.h:67-70,
     * concatenated: 4 x features inputs ("2x2 high-res neighbourhood"). */
    NTC_HIP_GRID_CONCAT2X2 = 1
} NtcHipGridMode;

typedef enum NtcHipWeightType {
    NTC_HIP_WEIGHTS_INT8 = 0, /* GenericInt8 blob, src/WeightLayout.cpp:42-49,184-247 */
    /* The reference's GenericFP8 blob (src/WeightLayout.cpp:51-71,249-262): e4m3 matrices and fp16
     * biases for the hidden layers, int8 + fp32 scale + int32 bias for the output layer - the weights
     * ITextureSet::Decompress takes unless asked for Int8 ones (src/TextureSet.cpp:1812,1826).
     * The arithmetic contract is the shader's, NtcEvaluateLayer / NtcSampleTextureSet_CoopVec_FP8 of
     * include/libntc/shaders/InferenceCoopVec.hlsli:22-124,127-160,235-398, with exact dot products:
     * e4m3-rounded fp16 inputs and activations, fp16 bias, HGELU-clamp in fp16, int8 output layer with fp32
     * scale and int32 bias fed by rne(80 y - 113).  It is NOT the bit pattern of cuda::Inference
     * (src/Inference.cu:65-100 through src/tin: FP16 tensor-core products with half accumulation, the last
     * hidden layer requantised as hrint(y * invStep) * step in fp16, an fp16 output layer, optimalToLinear
     * applied after the Inf/NaN test, src/tin/tin_activation.h:86-103): neither that kernel's nor the
     * driver's cooperative-vector accumulation order is defined, so equality with the reference's own
     * bits is unpinned for this network (the contract's tolerance for it is 1e-3 / 1 unorm8 step); the
     * only checker is this repository's restatement of the shader.  Known differences in corner cases:
     * an activation input of -Inf gives -0 here (max(x, -3) first) where the CUDA path propagates NaN
     * and stores 0; the two NaN encodings of an e4m3 weight decode as 0; the output layer is the
     * shader's int8 one, not fp16.  Decoded by ntc_hip_decode and ntc_hip_decode_queries for the
     * LibNTC 0.9.2 geometry (both grids bilinear 4-bit with 4 / 8 / 12 / 16 features, MLP 48-64-48-32-16). */
    NTC_HIP_WEIGHTS_FP8  = 1,
    /* Laid out exactly like NTC_HIP_WEIGHTS_INT8, but the bytes of the three hidden-layer matrices
     * are OCP e4m3 values w.  A hidden layer computes acc = bias_i32 + sum(512*w * in) exactly in
     * int32 (the result of an fp32-accumulating dot product without its rounding noise), then
     * r = float(acc) * scale as in the int8 path, so `scale` is per unit of w/512.  Inputs and
     * activations stay int8.  NaN encodings decode as 0. */
    NTC_HIP_WEIGHTS_FP8_SCALED = 2
} NtcHipWeightType;

typedef enum NtcHipOutputFormat {
    /* LibNTC's internal texture layout (src/ImageProcessing.h:20-33, src/RegressionKernels.h:36-45):
     * fp16, per row groups of two channels, element index
     *   y*W*C + (ch & ~1)*W + 2*x + (ch & 1),  C = channels rounded up to even. */
    NTC_HIP_OUT_FP16_PLANAR_PAIRS = 0,
    /* Pitch-linear pixels, all channels of a pixel together, fp16 (ChannelFormat::FLOAT16
     * of src/ImageProcessing.cu:141-164). */
    NTC_HIP_OUT_FP16_PIXELS  = 1,
    /* Pitch-linear pixels, unorm8 (ChannelFormat::UNORM8, same function). */
    NTC_HIP_OUT_UNORM8_PIXELS = 2
} NtcHipOutputFormat;

/* Geometry and arithmetic of one decoder.  The mounted LibNTC 0.9.2 is the preset
 * {16,4,BILINEAR,16, 16,4,BILINEAR,16, 3, 2, 48, {64,48,32}, 16, INT8}. */
typedef struct NtcHipDecoderSpec {
    int32_t hrFeatures;      /* features stored per high-res cell                         */
    int32_t hrBits;          /* bits per stored feature: 2 or 4 (16/bits features per u16) */
    int32_t hrMode;          /* NtcHipGridMode                                             */
    int32_t hrFeatureSlots;  /* input slots reserved per sampled cell (>= hrFeatures)      */
    int32_t lrFeatures;
    int32_t lrBits;
    int32_t lrMode;
    int32_t lrFeatureSlots;
    int32_t posEncWaves;     /* NTC_MLP_POS_ENC_WAVES = 3 -> 12 inputs                     */
    int32_t lodInputs;       /* 2 = the (lod, lod) pair of Inference.hlsli:117-119; 0 = none */
    int32_t inputChannels;   /* padded input width, multiple of 16, <= 64                  */
    int32_t hiddenChannels[NTC_HIP_MLP_LAYERS - 1];
    int32_t outputChannels;  /* 16                                                         */
    int32_t weightType;      /* NtcHipWeightType                                           */
} NtcHipDecoderSpec;

/* Byte offsets of the pieces of a weight blob (src/WeightLayout.h:33-50). */
typedef struct NtcHipWeightLayout {
    uint32_t weightOffset[NTC_HIP_MLP_LAYERS];
    uint32_t scaleOffset[NTC_HIP_MLP_LAYERS];  /* fp32 per output channel; unused (0) for fp8 hidden layers */
    uint32_t biasOffset[NTC_HIP_MLP_LAYERS];   /* int32 (int8 layers) or fp16 (fp8 hidden layers) */
    uint32_t bufferSize;
} NtcHipWeightLayout;

/* One colour mip: the fields of InferenceKernelParams that vary per launch
 * (src/RegressionCommon.h:55-80, filled at src/TextureSet.cpp:1806-1829). */
typedef struct NtcHipMipDesc {
    int32_t  width, height;          /* referenceWidth / referenceHeight                */
    int32_t  hrWidth, hrHeight;      /* highResLatentWidth / Height                     */
    int32_t  lrWidth, lrHeight;      /* lowResLatentWidth / Height                      */
    float    positionScale;          /* src/TextureSet.cpp:460                          */
    float    positionLod;            /* src/TextureSet.cpp:461; FP8 network: |lod| <= 3 */
    uint64_t hrOffset;               /* byte offset of the grid's first u16 layer in `latents` */
    uint64_t lrOffset;
    uint64_t outOffset;              /* byte offset of this mip in `output`             */
    uint64_t outRowPitch;            /* bytes between rows, pixel formats only          */
} NtcHipMipDesc;

/* One texture set to decode.  A latent grid is stored as in the NTC file:
 * ceil(features / (16/bits)) layers of height*width little-endian u16, layer after
 * layer (src/FeatureGridHost.h:92-93, src/Quantizer.cu:519-526); feature f of a cell
 * sits in layer f / (16/bits) at bits [bits*(f % (16/bits)), +bits). */
typedef struct NtcHipTextureSet {
    NtcHipDecoderSpec spec;
    int32_t  numMips;
    int32_t  numChannels;            /* channels written; outputs >= numChannels are dropped (Inference.cu:131) */
    int32_t  outputFormat;           /* NtcHipOutputFormat */
    int32_t  outPixelStride;         /* bytes between pixels, pixel formats only */
    const void* latents;             /* device */
    const void* weights;             /* device, blob laid out per ntc_hip_weight_layout() */
    void*       output;              /* device */
    uint64_t latentsBytes;           /* sizes of the three buffers; every grid, the blob and every */
    uint64_t weightsBytes;           /* mip's output extent are checked against them before launch */
    uint64_t outputBytes;
    NtcHipMipDesc mips[NTC_HIP_MAX_MIPS];
    const void* queryLatents;        /* device, optional: the grids once more in query order, see      */
    uint64_t queryLatentsBytes;      /* ntc_hip_build_query_latents; used by ntc_hip_decode_queries only */
} NtcHipTextureSet;

/* ---- library / device ------------------------------------------------------------ */

/* A context: one device, one stream (opaque). */
typedef struct NtcHipContext NtcHipContext;
/* Creates a context on HIP device `device` (which must be a gfx950 device) with a stream of its own.
 * Replaces the reference's cudaSetDevice + cudaInitDevice in CreateContext (src/PublicFunctions.cpp:84-112). */
int ntc_hip_create(int device, NtcHipContext** outContext);
/* Waits for the context's work, then releases its stream and working memory.  Memory from
 * ntc_hip_ctx_alloc is the caller's to free first. */
void ntc_hip_destroy(NtcHipContext* context);

/* Creates the default context (the one behind every function below that takes no context) on `device`
 * and makes that device current; a second call with another device replaces it. */
int ntc_hip_init(int device);
void ntc_hip_shutdown(void);
/* Message of the last failed call on this thread ("" if none). GetLastErrorMessage, include/libntc/ntc.h:1331. */
const char* ntc_hip_last_error(void);
/* Name, compute-unit count of the initialised device. */
int ntc_hip_device_info(char* name, size_t nameSize, int* computeUnits);
/* Peak engine clock of the initialised device in kHz (hipDeviceProp_t::clockRate), for ceilings that are
 * quoted per clock. */
int ntc_hip_device_clock(int* clockRateKHz);

/* ---- memory (DeviceArray<T> of src/CudaArray.h:104-181) --------------------------- */
int ntc_hip_alloc(void** devPtr, size_t bytes);
int ntc_hip_free(void* devPtr);
int ntc_hip_upload(void* dst, const void* src, size_t bytes);     /* host -> device, synchronous */
int ntc_hip_download(void* dst, const void* src, size_t bytes);   /* device -> host, synchronous */
int ntc_hip_memset(void* dst, int value, size_t bytes);
int ntc_hip_synchronize(void);

/* ---- layout helpers (host only, no device needed) --------------------------------- */

/* Offsets of a weight blob for `spec`: MakeQuantizedWeightLayout, src/WeightLayout.cpp:142-268. */
int ntc_hip_weight_layout(const NtcHipDecoderSpec* spec, NtcHipWeightLayout* outLayout);
/* Bytes one latent grid of the given shape occupies. */
uint64_t ntc_hip_grid_bytes(int32_t width, int32_t height, int32_t features, int32_t bits);

/* ---- the hot path ----------------------------------------------------------------- */

/* Decodes every mip of every set in ONE launch on the library stream (asynchronous).
 * Replaces the per-mip loop over cuda::Inference of src/TextureSet.cpp:1782-1831. */
int ntc_hip_decode(const NtcHipTextureSet* sets, int32_t numSets);

/* Same work, repeated `iterations` times between two HIP events on the library stream;
 * returns the mean milliseconds of one repetition (the reference's own timer brackets the
 * same region with cudaEvents, src/TextureSet.cpp:1772-1882).  Synchronous. */
int ntc_hip_decode_timed(const NtcHipTextureSet* sets, int32_t numSets, int32_t iterations,
                         float* outMillisecondsPerIteration);

/* Device time of a sequence of calls: ntc_hip_timer_begin records a HIP event on the context's stream, ntc_hip_timer_end
 * records a second one behind everything queued since, waits for it and returns the milliseconds between the two.
 * This is how the reference times its own decompression (cudaEventRecord around the per-mip loop,
 * src/TextureSet.cpp:1772-1779,1866-1882); ntc_hip_decode_timed is the special case of one decode repeated.
 * One span at a time per context; _end without _begin: NTC_HIP_ERR_INVALID_ARG.  _end is synchronous. */
int ntc_hip_timer_begin(void);
int ntc_hip_timer_end(float* outMilliseconds);

/* ntc_hip_decode for callers that cannot allocate device memory: code under HIP graph capture, serving
 * loops and harnesses that forbid hipMalloc.  No counterpart in the reference.  ntc_hip_decode keeps its
 * mip table in device memory that it allocates (and grows) on demand and fills through pinned staging
 * memory; here the table lives in an array built into the library's code object, NTC_HIP_STATIC_TABLE_MIPS
 * entries and one more 256-byte line (about 34 KB, held by every GPU the library runs on until the process
 * ends), and travels to the device as kernel arguments; the extra line holds the word through which the first of
 * the FP8 network's two launches tells the second whether a set is left for it.  The call allocates nothing on the device or the host (the table is assembled
 * in an array inside the context), frees nothing and copies nothing: it launches
 * one small table-writing kernel per 16 mips and then the decode kernel of ntc_hip_decode, same results.
 * More than NTC_HIP_STATIC_TABLE_MIPS mips over all sets of one call: NTC_HIP_ERR_INVALID_ARG.
 * All calls on one GPU, from whatever context, share that GPU's array, which keeps the last call's table.
 * Calls queued on ONE context's stream run in order and are safe; calls that overlap on one GPU - from
 * two contexts, whose streams are not ordered against each other, or from threads of one process without
 * the serialisation this library asks for - race on it.  Asynchronous on the context's stream. */
#define NTC_HIP_STATIC_TABLE_MIPS 256
int ntc_hip_decode_static(const NtcHipTextureSet* sets, int32_t numSets);

/* Random-access decode: "inference on sample", NtcSampleTextureSet of
 * include/libntc/shaders/Inference.hlsli:282-357, for a list of sample points instead of a
 * shader invocation.  Query i decodes texel (floor(u*W), floor(v*H)) of colour mip `mip`
 * (clamped to the image, as the reference clamps out-of-bounds texels) and writes its 16
 * network outputs as fp16 at out + 32*i.  A mip index outside the set writes zeros (the
 * reference returns false and leaves the outputs alone).  The set's output fields are not
 * used.  Queries and out are device memory.  Asynchronous / timed like ntc_hip_decode. */
typedef struct NtcHipQuery { float u, v; int32_t mip; } NtcHipQuery;
int ntc_hip_decode_queries(const NtcHipTextureSet* set, const NtcHipQuery* queries, uint64_t numQueries,
                           void* out, uint64_t outBytes);
int ntc_hip_decode_queries_timed(const NtcHipTextureSet* set, const NtcHipQuery* queries, uint64_t numQueries,
                                 void* out, uint64_t outBytes, int32_t iterations,
                                 float* outMillisecondsPerIteration);

/* A second copy of a set's latent grids laid out for scattered sample points.  In the file layout a
 * grid is ceil(features/4) separate layers, so the 2 x 2 cells a sample point needs lie in 8 different
 * cache lines per grid; here a grid is cut into bricks of 4 x 4 cells (8 x 8 for one-layer grids) that
 * hold all layers of their cells together, [cell row][cell column][layer], one 128-byte line per brick
 * for four layers, and a sample point touches 1.6 lines per grid on average.  No reference counterpart
 * (the reference samples a hardware texture there, Inference.hlsli:62-87).
 * ntc_hip_query_latents_bytes: size of that copy for the set's geometry (0 on a malformed set).
 * ntc_hip_build_query_latents: fills dst (device, 128-byte aligned) from set->latents; asynchronous on
 * the library stream.  Put dst into set->queryLatents / queryLatentsBytes for ntc_hip_decode_queries;
 * results are the same bits with or without it. */
uint64_t ntc_hip_query_latents_bytes(const NtcHipTextureSet* set);
int ntc_hip_build_query_latents(const NtcHipTextureSet* set, void* dst, uint64_t dstBytes);

/* Extracts channels of one decoded mip from the internal fp16 layout into a user image:
 * what ITextureSet::ReadChannels does through cuda::CopyImage (src/TextureSet.cpp:915-985,
 * src/ImageProcessing.cu:24-72,86-164,220-277).  When dstWidth x dstHeight differs from the mip's size the
 * image is resampled with the reference's bilinear filter (edge texels clamped, taps of zero weight
 * not read; a 2x reduction is a 2x2 box filter).  Each copied channel is decoded from its storage colour space and encoded into the
 * destination's (0 linear, 1 sRGB, 2 HLG; src/CudaUtils.h:61-114); with useDithering every
 * destination channel of UNORM formats gets the reference's hash-based noise of +-1/2 step
 * (src/CudaUtils.h:117-184).  Destination channels beyond numChannels get the reference's
 * defaults (alpha 1, others 0).  Asynchronous on the library stream. */
typedef struct NtcHipReadChannels {
    const void* planarPairs;    /* device: start of the mip, NTC_HIP_OUT_FP16_PLANAR_PAIRS layout */
    uint64_t    planarBytes;    /* bytes available from planarPairs */
    int32_t     width, height;  /* of the mip */
    int32_t     setChannels;    /* channel count of the set, even */
    int32_t     firstChannel, numChannels;
    void*       dst;            /* device */
    uint64_t    dstBytes;
    int32_t     format;         /* ChannelFormat of include/libntc/ntc.h:227-236: 1 UNORM8, 2 UNORM16, 3 FLOAT16, 4 FLOAT32, 5 UINT32 */
    int32_t     useDithering;
    uint64_t    pixelStride, rowPitch;
    uint8_t     srcColorSpaces[16];   /* storage colour space of set channel firstChannel + i */
    uint8_t     dstColorSpaces[16];   /* colour space wanted for copied channel i */
    int32_t     dstWidth, dstHeight;  /* size of the user image; 0, 0 = the mip's size */
} NtcHipReadChannels;
int ntc_hip_read_channels(const NtcHipReadChannels* params);

/* Stores a user image into the internal fp16 layout of one mip: what ITextureSet::WriteChannels
 * does through cuda::CopyImage (src/TextureSet.cpp:829-913, src/ImageProcessing.cu:107-164,220-277).
 * A source image of another size (srcWidth x srcHeight) is resampled as in NtcHipReadChannels; colour
 * spaces as there.  Asynchronous on the library stream. */
typedef struct NtcHipWriteChannels {
    const void* src;            /* device: pitch-linear user image */
    uint64_t    srcBytes;
    int32_t     format;         /* ChannelFormat, as in NtcHipReadChannels */
    int32_t     verticalFlip;
    uint64_t    pixelStride, rowPitch;
    void*       planarPairs;    /* device: start of the mip in the internal layout */
    uint64_t    planarBytes;
    int32_t     width, height, setChannels, firstChannel, numChannels, reserved;
    uint8_t     srcColorSpaces[16];   /* colour space of channel i of the user image */
    uint8_t     dstColorSpaces[16];   /* storage colour space of set channel firstChannel + i */
    int32_t     srcWidth, srcHeight;  /* size of the user image; 0, 0 = the mip's size */
} NtcHipWriteChannels;
int ntc_hip_write_channels(const NtcHipWriteChannels* params);

/* Resamples one image of the internal layout into another (all channels), decoding each channel from
 * its storage colour space, filtering, and encoding it again: cuda::ResizeMultichannelImage as
 * ITextureSet::GenerateMips uses it from one mip to the next (src/ImageProcessing.cu:178-218,
 * src/TextureSet.cpp:1121-1142).  The images must not overlap.  Asynchronous on the library stream. */
int ntc_hip_resize_planar(const void* srcPlanarPairs, uint64_t srcBytes, int32_t srcWidth, int32_t srcHeight,
                          void* dstPlanarPairs, uint64_t dstBytes, int32_t dstWidth, int32_t dstHeight,
                          int32_t setChannels, const uint8_t* channelColorSpaces /* 16 */);

/* Mean squared error per channel between two images in the internal layout (a decoded mip and its
 * reference): the loss branch of InferenceKernel + ReduceLoss (src/Inference.cu:77-118,142-156,
 * src/Optimizer.cu:335-390) as a pass of its own.  Channels whose bit is clear in validChannelMask
 * report 0.  maskChannelIndex / discardMaskedOutPixels are the alpha-mask options of
 * ITextureSet::SetMaskChannelIndex (include/libntc/ntc.h:936-940): with an index >= 0 the DECODED mask
 * channel is clamped to [0, 1] in place before it is compared (Inference.cu:96-97), and with the
 * discard flag texels whose reference mask value is zero count on the mask channel only
 * (Inference.cu:80-84,107-108).  A negative index means no mask channel; the decoded image is then only
 * read.  outMse receives 16 floats.  Synchronous. */
int ntc_hip_image_loss(void* decodedPlanarPairs, const void* referencePlanarPairs, uint64_t planarBytes,
                       int32_t width, int32_t height, int32_t setChannels, uint32_t validChannelMask,
                       int32_t maskChannelIndex, int32_t discardMaskedOutPixels, float* outMse);

/* One image of an image-difference pass: pitch-linear pixels of 1..4 channels (R, G, B, A) in one
 * of the ChannelFormat encodings; channels a pixel does not store read as 0, 0, 0, 1. */
typedef struct NtcHipImage {
    const void* data;           /* device */
    uint64_t    bytes;
    uint64_t    pixelStride, rowPitch;
    int32_t     width, height;  /* size of the whole image (the compared extent must lie inside) */
    int32_t     format;         /* ChannelFormat, as in NtcHipReadChannels */
    int32_t     numChannels;
} NtcHipImage;

/* Per-channel mean squared error (or mean squared log error) between the same rectangle of two
 * images: the compute pass IContext::MakeImageDifferenceComputePass describes
 * (include/libntc/ntc.h:1103-1121,1227-1239, src/shaders/ImageDifference.hlsl, constants
 * include/libntc/shaders/ImageDifferenceConstants.h).  Every workgroup covers 64 x 64 pixels, divides
 * its four sums by width * height and ADDS them, as 16.48 fixed point, to the four uint64 at
 * output + outputOffset, which the caller clears beforehand; ntc::DecodeImageDifferenceResult turns
 * them into doubles.  With useAlphaThreshold, pixels whose alpha is below the threshold in both
 * images contribute to the alpha channel only; with useMSLE the compared values are log(|v| + 1).
 * The order in which a workgroup adds its pixels is not defined by the reference (wave intrinsics);
 * here it is fixed, so results are reproducible.  Asynchronous on the library stream. */
typedef struct NtcHipImageDifference {
    NtcHipImage a, b;
    int32_t     left, top, width, height;     /* extent compared in both images */
    float       alphaThreshold;
    int32_t     useAlphaThreshold;
    int32_t     useMSLE;
    uint32_t    outputOffset;                 /* bytes, multiple of 8 */
    void*       output;                       /* device */
    uint64_t    outputBytes;
} NtcHipImageDifference;
int ntc_hip_image_difference(const NtcHipImageDifference* params);

/* BC1 .. BC7 compression of an image: the block-compression compute pass of
 * IContext::MakeBlockCompressionComputePass for those formats (include/libntc/ntc.h:1050-1100,
 * src/shaders/CompressBC1.hlsl .. CompressBC7.hlsl, src/shaders/BlockCompressCommon.hlsli).
 * widthInBlocks x heightInBlocks blocks of 4 x 4 pixels starting at (srcLeft, srcTop) are encoded and
 * stored row-major with dstRowPitch bytes per row of blocks, the first at block (dstOffsetX, dstOffsetY).
 * dstFormat is a BlockCompressedFormat:
 *   1  BC1, 8 bytes per block, from R, G, B and A (pixels with A <= alphaThreshold may become transparent);
 *   2  BC2, 16 bytes: 4-bit alpha, then a BC1 colour block;
 *   3  BC3, 16 bytes: a BC4 block of A, then a BC1 colour block;
 *   4  BC4, 8 bytes, from R;      5  BC5, 16 bytes, from R then G;
 *   7  BC7, 16 bytes, from R, G, B and A (src/shaders/CompressBC7.hlsl); see modeBuffer below.  The
 *      reference's BC7 shader ignores dstOffsetInBlocks (CompressBC7.hlsl:1590); here it is honoured as for
 *      the other formats;
 *   6  BC6H, unsigned half floats, 16 bytes, from R, G and B clamped to [0, 65504] (src/shaders/CompressBC6.hlsl);
 * Channels the image does not have read as 0 (alpha as 1); pixels outside the image read as 0 in every
 * channel, like a texture load there.  Asynchronous on the library stream. */
typedef struct NtcHipBlockCompress {
    NtcHipImage src;
    int32_t     srcLeft, srcTop;
    int32_t     widthInBlocks, heightInBlocks;
    int32_t     dstFormat;
    int32_t     dstOffsetX, dstOffsetY;       /* in blocks */
    float       alphaThreshold;               /* BC1 only; the reference's default is 1 / 255 */
    void*       dst;                          /* device, 8-byte aligned */
    uint64_t    dstBytes;
    uint64_t    dstRowPitch;                  /* bytes per row of blocks, multiple of 8 */
    /* BC7 only: the mode buffer of MakeBC7ModeBuffer (include/libntc/ntc.h:1381-1391), 9 bits per block of a
     * modeMapWidthInBlocks x modeMapHeightInBlocks map; the block (x, y) of this call uses the entry at
     * (x + modeMapOffsetX, y + modeMapOffsetY).  Then only that mode and partition are encoded (several times
     * faster); a block with no entry becomes the reference's marker block of four coloured squares.  NULL:
     * every mode is tried. */
    const void* modeBuffer;                   /* device, 4-byte aligned */
    uint64_t    modeBufferBytes;
    uint64_t    modeBufferByteOffset;         /* multiple of 4 */
    int32_t     modeMapWidthInBlocks, modeMapHeightInBlocks;
    int32_t     modeMapOffsetX, modeMapOffsetY;
} NtcHipBlockCompress;
int ntc_hip_block_compress(const NtcHipBlockCompress* params);

/* ---- every entry point above on a context of the caller's (same arguments, same results) ------------ */
int ntc_hip_ctx_device_info(NtcHipContext* context, char* name, size_t nameSize, int* computeUnits);
int ntc_hip_ctx_device_clock(NtcHipContext* context, int* clockRateKHz);
int ntc_hip_ctx_alloc(NtcHipContext* context, void** devPtr, size_t bytes);
int ntc_hip_ctx_free(NtcHipContext* context, void* devPtr);
int ntc_hip_ctx_upload(NtcHipContext* context, void* dst, const void* src, size_t bytes);
int ntc_hip_ctx_download(NtcHipContext* context, void* dst, const void* src, size_t bytes);
int ntc_hip_ctx_memset(NtcHipContext* context, void* dst, int value, size_t bytes);
int ntc_hip_ctx_synchronize(NtcHipContext* context);
int ntc_hip_ctx_decode(NtcHipContext* context, const NtcHipTextureSet* sets, int32_t numSets);
int ntc_hip_ctx_decode_static(NtcHipContext* context, const NtcHipTextureSet* sets, int32_t numSets);
int ntc_hip_ctx_timer_begin(NtcHipContext* context);
int ntc_hip_ctx_timer_end(NtcHipContext* context, float* outMilliseconds);
int ntc_hip_ctx_decode_timed(NtcHipContext* context, const NtcHipTextureSet* sets, int32_t numSets, int32_t iterations, float* outMs);
int ntc_hip_ctx_build_query_latents(NtcHipContext* context, const NtcHipTextureSet* set, void* dst, uint64_t dstBytes);
int ntc_hip_ctx_decode_queries(NtcHipContext* context, const NtcHipTextureSet* set, const NtcHipQuery* queries, uint64_t numQueries, void* out, uint64_t outBytes);
int ntc_hip_ctx_decode_queries_timed(NtcHipContext* context, const NtcHipTextureSet* set, const NtcHipQuery* queries, uint64_t numQueries, void* out, uint64_t outBytes, int32_t iterations, float* outMillisecondsPerIteration);
int ntc_hip_ctx_read_channels(NtcHipContext* context, const NtcHipReadChannels* p);
int ntc_hip_ctx_write_channels(NtcHipContext* context, const NtcHipWriteChannels* p);
int ntc_hip_ctx_image_loss(NtcHipContext* context, void* decoded, const void* reference, uint64_t planarBytes, int32_t width, int32_t height, int32_t setChannels, uint32_t validChannelMask, int32_t maskChannelIndex, int32_t discardMaskedOutPixels, float* outMse);
int ntc_hip_ctx_resize_planar(NtcHipContext* context, const void* src, uint64_t srcBytes, int32_t srcWidth, int32_t srcHeight, void* dst, uint64_t dstBytes, int32_t dstWidth, int32_t dstHeight, int32_t setChannels, const uint8_t* channelColorSpaces);
int ntc_hip_ctx_image_difference(NtcHipContext* context, const NtcHipImageDifference* p);
int ntc_hip_ctx_block_compress(NtcHipContext* context, const NtcHipBlockCompress* p);

/* Self-check of the MFMA operand layout the kernels assume: multiplies a 16x64 by a
 * 64x16 int8 matrix on the device (row-major host arrays), writes the 16x16 int32
 * product.  No reference counterpart; used by the tests. */
int ntc_hip_selftest_mfma(const int8_t* a16x64, const int8_t* b64x16, int32_t* d16x16);

/* Same for the fp16 MFMA the hidden layers use when every partial sum of a layer stays an integer
 * below 2^24: D = A*B + C, A 16 x depth and B depth x 16 as row-major IEEE halves, C and D 16x16
 * floats, depth 16 or 32.  With integer-valued operands of that size the result must be the
 * exact integer, whatever order the hardware adds in.  No reference counterpart; used by the tests. */
int ntc_hip_selftest_mfma_f16(const uint16_t* aHalves, const uint16_t* bHalves, const float* c16x16, float* d16x16, int32_t depth);

/* The fp16 primitives of the FP8 network's activation stage applied to `count` halves (at most 2^20):
 * out[0..count) the HGELU-clamp of each input, out[count..2 count) each input rounded to e4m3 (as a half),
 * out[2 count..3 count) 80 x - 113 rounded to an integer (as a half; defined for inputs in [-0.1875, 3]).
 * No reference counterpart; used by the tests. */
int ntc_hip_selftest_fp8_activation(const uint16_t* halves, int32_t count, uint16_t* out);

#ifdef __cplusplus
}
#endif
#endif /* NTC_HIP_H */
