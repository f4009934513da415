/*
 * C ABI of the MI355X (gfx950) skip-gram negative-sampling library.
 *
 * The first four functions are the drop-in boundary: they have the parameter lists of the
 * reference's GPU operator launchers (jni/include/MatKernel.hpp:77,79,83,85), which its JNI glue
 * (jni/src/BIDMach_CUMACH.cpp:434-493) calls on behalf of edu.berkeley.bid.CUMACH
 * (src/main/java/edu/berkeley/bid/CUMACH.java:90,92,96,98).  Every pointer is a device pointer
 * owned by the caller; the library never allocates, frees or keeps them.
 *
 * Layout: A and B are nrows x vocab, column-major, fp32: word w's vector is the contiguous run
 * [w*nrows, (w+1)*nrows).  Word ids are int32.
 *
 * Error convention (reference: jni/src/DNN127.cu:1417-1419): 0 on success, otherwise the
 * hipError_t value.  A shape or argument the library rejects returns hipErrorInvalidValue (1),
 * as the reference's launchers return 1 for a shape they have no kernel for
 * (DNN127.cu:1397,1414-1415,1435).  The library never aborts the process.
 *
 * Threading (reference: MatKernel.hpp:2 and the per-thread default stream of its build): the
 * four reference calls block until the work is done.  Each host thread has its own launch stream
 * (one the library creates on the thread's first call on a device, ordered with the legacy
 * default stream as the reference's per-thread default streams are, jni/src/configure:158,196;
 * w2v_set_stream replaces it) and its own Eval scratch buffer, so calls from two threads overlap
 * on the device.
 */
#ifndef BIDMACH_W2V_H_
#define BIDMACH_W2V_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- The reference operator API -------------------------------------------------------- */

/* Replaces word2vecPos, MatKernel.hpp:77 / DNN127.cu:1389-1420; arithmetic of
 * BIDMach_CPUMACH.c:10-78.  ncols tokens; token i with W[i] >= 0 is a centre word whose window
 * is the offsets j in [LB[i], UB[i]], j != 0, 0 <= i+j < ncols, W[i+j] >= 0.  A is indexed by the
 * centre word, B by the context word; both are updated in place.  `shift` is the caller's maximum
 * window half-width (the reference's template selector, Word2Vec.scala:373 passes nskip); here
 * it only sizes the halo a tile of tokens stages on chip, so any value gives the same result and
 * any window width works. */
int word2vecPos(int nrows, int ncols, int shift, int *W, int *LB, int *UB, float *A, float *B,
                float lrate, float vexp);

/* Replaces word2vecNeg, MatKernel.hpp:79 / DNN127.cu:1423-1452; arithmetic of
 * BIDMach_CPUMACH.c:186-264.  ncols groups; group i pairs the nwa words WA[i*nwa + j] (columns of
 * A) with the nwb words WB[i*nwb + k] (columns of B).  Any nwa and nwb (see w2v_max_nwb). */
int word2vecNeg(int nrows, int ncols, int nwa, int nwb, int *WA, int *WB, float *A, float *B,
                float lrate, float vexp);

/* Replaces word2vecNegFilt, MatKernel.hpp:81 / DNN127.cu:670-823,1454-1483 (CUMACH.java:94; used by
 * the reference when only the first `nwords` columns of a larger model are resident on the GPU,
 * Word2Vec.scala:448).  As word2vecNeg, but a word id >= nwords is skipped together with every
 * pair it takes part in (DNN127.cu:690-711); A and B hold nwords columns. */
int word2vecNegFilt(int nrows, int ncols, int nwords, int nwa, int nwb, int *WA, int *WB, float *A,
                    float *B, float lrate, float vexp);

/* Sliced, multi-part models.  Device counterparts of the reference's CPU-only
 * CPUMACH.word2vecPosSlice / word2vecNegSlice (CPUMACH.java:14,19; BIDMach_CPUMACH.c:80-184,
 * :267-366; dispatched from Word2Vec.scala:404-467) and of its Scala-only forward twins
 * evalPosCPUslice / evalNegCPUslice (Word2Vec.scala:1007-1069, :1134-1200).  Same argument lists
 * with the thread count dropped and the length of MM added (a C array has none).
 *
 * MM is a HOST array of nmats DEVICE pointers, the reference's modelmats: part m of the packed
 * model has its B table (nrows x maxCols, column-major) at MM[2m] and its A table at MM[2m+1];
 * with dualMode != 0 the parts start at MM[2] and MM[0], MM[1] are not touched.  At most
 * w2v_max_slice_parts() parts.  Word id w lives in packed column w if w < nHead, else
 * nHead + (w - nHead) / nslices, and is resident iff w < nHead or w % nslices == islice
 * (mapIndx, BIDMach_CPUMACH.c:80-88).  A pair is trained iff both words are resident and one of
 * them is a tail word of this slice, or both are head words and doHead > 1; a column is written
 * iff it is a tail word of this slice, or a head word and doHead > 0.  The forward twins score
 * the pairs whose two words are resident and ADD the sum into the device double Retval[0].
 * Deviation: inside a part the column is packed - (packed / maxCols) * maxCols for either value of
 * dualMode (the reference's expression, :87, points maxCols columns before the part when
 * dualMode is set). */
int word2vecPosSlice(int nrows, int ncols, int shift, int *W, int *LB, int *UB, float **MM,
                     int nmats, float lrate, float vexp, int islice, int nslices, int maxCols,
                     int nHead, int dualMode, int doHead);
int word2vecNegSlice(int nrows, int ncols, int nwa, int nwb, int *WA, int *WB, float **MM,
                     int nmats, float lrate, float vexp, int islice, int nslices, int maxCols,
                     int nHead, int dualMode, int doHead);
int word2vecEvalPosSlice(int nrows, int ncols, int shift, int *W, int *LB, int *UB, float **MM,
                         int nmats, int islice, int nslices, int maxCols, int nHead, int dualMode,
                         double *Retval);
int word2vecEvalNegSlice(int nrows, int ncols, int nwa, int nwb, int *WA, int *WB, float **MM,
                         int nmats, int islice, int nslices, int maxCols, int nHead, int dualMode,
                         double *Retval);
int w2v_max_slice_parts(void);

/* Replaces word2vecEvalPos, MatKernel.hpp:83 / DNN127.cu:1485-1516; arithmetic of
 * BIDMach_CPUMACH.c:368-427.  Adds sum(log(max(sigmoid(a.b), floor))) over the valid pairs into
 * the device float Retval[0] (the caller clears it first, Word2Vec.scala:476). */
int word2vecEvalPos(int nrows, int ncols, int shift, int *W, int *LB, int *UB, float *A, float *B,
                    float *Retval);

/* Replaces word2vecEvalNeg, MatKernel.hpp:85 / DNN127.cu:1519-1548; arithmetic of
 * BIDMach_CPUMACH.c:429-483.  Adds sum(log(max(1 - sigmoid(a.b), floor))) into Retval[0]. */
int word2vecEvalNeg(int nrows, int ncols, int nwa, int nwb, int *WA, int *WB, float *A, float *B,
                    float *Retval);

/* ---- Extensions with no counterpart in the reference's GPU API ------------------------- */

/* Same sums, added into a device double (the reference's CPU twins return jdouble,
 * BIDMach_CPUMACH.c:368,429; its GPU path keeps only a float). */
int word2vecEvalPosF64(int nrows, int ncols, int shift, int *W, int *LB, int *UB, float *A,
                       float *B, double *Retval);
int word2vecEvalNegF64(int nrows, int ncols, int nwa, int nwb, int *WA, int *WB, float *A,
                       float *B, double *Retval);

/* word2vecEvalNeg for callers that cannot allocate device memory (tight serving loops, harnesses
 * that forbid hipMalloc, hosts that score between the captures of a HIP graph).  It has no
 * counterpart in the reference.  Same arguments and the same result as word2vecEvalNeg (added
 * into the device float Retval[0]).  Like it, the call blocks until the sum is there (it ends in
 * a stream synchronisation), so it cannot itself be recorded into a graph.  The per-workgroup
 * partial sums go to a 64 KB array that is part of the library's device code instead of a buffer
 * taken from hipMalloc on a thread's first call, and the call makes no hipMalloc, hipFree or
 * other allocating call; it creates no stream either (it launches on the caller's stream, on the
 * thread's own if an earlier call made one, else on the legacy default stream).  At most w2v_no_alloc_max_groups()
 * (16,777,216) groups per call; more is rejected with hipErrorInvalidValue.  Every call on a GPU
 * uses that GPU's one array: calls that overlap in time on one GPU (from several threads or
 * streams) race and return wrong sums; one after the other they are independent (nothing in the
 * array carries over). */
int word2vecEvalNegNoAlloc(int nrows, int ncols, int nwa, int nwb, int *WA, int *WB, float *A,
                           float *B, float *Retval);
int w2v_no_alloc_max_groups(void);

/* Enqueue-only forms of the four operators: same arguments, same results, but they return after
 * the launch; completion is observed with w2v_synchronize() or a timer. */
int word2vecPosAsync(int nrows, int ncols, int shift, int *W, int *LB, int *UB, float *A, float *B,
                     float lrate, float vexp);
int word2vecNegAsync(int nrows, int ncols, int nwa, int nwb, int *WA, int *WB, float *A, float *B,
                     float lrate, float vexp);
int word2vecEvalPosAsync(int nrows, int ncols, int shift, int *W, int *LB, int *UB, float *A,
                         float *B, float *Retval);
int word2vecEvalNegAsync(int nrows, int ncols, int nwa, int nwb, int *WA, int *WB, float *A,
                         float *B, float *Retval);

/* Reduced-precision storage: the four operators on bfloat16 tables (A and B are nrows x vocab,
 * column-major, 2 bytes per element).  No counterpart in the reference, whose tables are fp32
 * throughout; the argument lists are those of the four operators above with the element type
 * changed, a seed added to the update calls and the forward sums added into a device double.
 * A column is widened to fp32 when it is read; dots, sigmoid, scales and deltas are the fp32
 * arithmetic of BIDMach_CPUMACH.c:10-78 / :186-264; a column is narrowed when it is written back,
 * with stochastic rounding (the magnitude rounds up with probability dropped-bits / 65536, so the
 * expectation of the stored value is the fp32 value) drawn from a counter-based generator keyed
 * by `seed`, the token / group index, the write inside it and the row: pass a new seed for every
 * call.  There is no floating-point atomic add on these tables: a write-back is a compare-and-swap
 * of the 4-byte word that holds the elements, repeated with the value found when another update
 * got there first, so concurrent updates of one column are all kept (a plain store of
 * "value read + delta" loses most updates of the frequent words once thousands of work units are
 * in flight).  With an odd nrows or a table on an odd 2-byte boundary the word that holds the
 * first or last element of a table reaches 2 bytes outside it; those bytes are written back
 * unchanged and must be addressable (they are inside any allocation the table is a view of).
 * nwb <= w2v_max_nwb(); an update of groups with more than 8 B words needs nwa <= 5, or nwa <= 16
 * with nrows <= 512 (hipErrorInvalidValue otherwise), and runs on a few hundred wavefronts. */
int word2vecPosBf16(int nrows, int ncols, int shift, int *W, int *LB, int *UB, unsigned short *A,
                    unsigned short *B, float lrate, float vexp, unsigned long long seed);
int word2vecNegBf16(int nrows, int ncols, int nwa, int nwb, int *WA, int *WB, unsigned short *A,
                    unsigned short *B, float lrate, float vexp, unsigned long long seed);
/* Enqueue-only forms of the two update calls (completion: w2v_synchronize() or a timer). */
int word2vecPosBf16Async(int nrows, int ncols, int shift, int *W, int *LB, int *UB,
                         unsigned short *A, unsigned short *B, float lrate, float vexp,
                         unsigned long long seed);
int word2vecNegBf16Async(int nrows, int ncols, int nwa, int nwb, int *WA, int *WB,
                         unsigned short *A, unsigned short *B, float lrate, float vexp,
                         unsigned long long seed);
int word2vecEvalPosBf16(int nrows, int ncols, int shift, int *W, int *LB, int *UB,
                        unsigned short *A, unsigned short *B, double *Retval);
int word2vecEvalNegBf16(int nrows, int ncols, int nwa, int nwb, int *WA, int *WB,
                        unsigned short *A, unsigned short *B, double *Retval);
/* Number of frequent words (ids 0 .. n-1; ids are frequency ranks) whose bf16 columns are updated
 * through an fp32 side buffer during a call: readers add table and side buffer in fp32, writers
 * add their delta to the side buffer with float atomics, and the end of the call narrows the sum
 * back into the table with one stochastic rounding per element (slot: unit 0xFFFFFFFF of the
 * generator).  A compare-and-swap on a column that thousands of work units update at once fails
 * nearly every time; float atomics need no retry.  Default 1024, at most 4096, 0 = every column
 * by compare-and-swap.  Process-wide; the side buffers belong to the calling thread. */
int w2v_set_bf16_hot_words(int n);
int w2v_get_bf16_hot_words(void);

/* Whole-table conversions between device buffers of n elements: fp32 -> bf16 rounds to nearest
 * (ties to even), bf16 -> fp32 is exact.  Blocking. */
int w2v_f32_to_bf16(size_t n, const float *src, unsigned short *dst);
int w2v_bf16_to_f32(size_t n, const unsigned short *src, float *dst);

/* Floor inside the Eval logarithms, process-wide.  Default 1e-40 (BIDMach_CPUMACH.c:409,467);
 * the reference's Scala and CUDA twins use 1e-20 (Word2Vec.scala:995,1123; DNN127.cu:310,916). */
void w2v_set_eval_floor(double floor_value);
double w2v_get_eval_floor(void);

/* Launch stream of the calling thread.  w2v_set_stream: a hipStream_t passed as void* (NULL = the
 * legacy default stream); w2v_reset_stream: back to the thread's own stream; w2v_get_stream: the
 * stream the next call will launch on (creates the thread's own stream if there is none yet). */
int w2v_set_stream(void *stream);
int w2v_reset_stream(void);
void *w2v_get_stream(void);
int w2v_synchronize(void);

/* Frees the device scratch memory the calling thread holds (per device: the forward sums'
 * partial buffer, the shadow and occurrence-count buffers of the update operators, the fp32 side
 * buffers of the bfloat16 operators; allocated on the thread's first calls) and destroys the
 * thread's own launch streams, after waiting for them.  The next call allocates it again.  Call it before a worker thread that
 * used the library ends (a JVM thread pool, say): thread-local scratch is not freed by thread
 * exit.  No counterpart in the reference, whose launchers keep no state. */
int w2v_release_thread(void);

/* Upper bound on the workgroups of the two update kernels, process-wide (0 = as many as the
 * device holds, the default).  The update kernels are persistent: each workgroup walks a
 * contiguous range of the minibatch in order, so this bounds the number of work units in flight
 * and with it how stale a Hogwild read can be (the reference's CPU path bounds it by its thread
 * count, BIDMach_CPUMACH.c:21-24). */
int w2v_set_max_workgroups(int n);
int w2v_get_max_workgroups(void);

/* Ordered form of word2vecPos / word2vecNeg / word2vecNegFilt, of word2vecPosSlice /
 * word2vecNegSlice and of word2vecPosBf16 / word2vecNegBf16, process-wide.  The reference's CPU
 * path keeps as many work units in flight as it has threads (BIDMach_CPUMACH.c:21-24, :197-201),
 * each of which reads a column just before it uses it and writes a B column back before it
 * reads the next (:57-61, :244-246).  On a raw (not subsampled) Zipf stream, where a tenth of
 * all tokens are the most frequent word, training at the reference's step size is at the edge
 * of stability and its result depends on how many updates of the frequent words a reader
 * misses; thousands of work units in flight, or a tile of adjacent tokens working from one
 * snapshot, then end many percent away from the reference's held-out loss.  In the ordered form
 * a few hundred wavefronts each walk a contiguous range of tokens / groups in the reference's
 * order, with every column read afresh and every B delta added before the next read.
 *  -1  (default) decided per launch on the device, by the same count that decides about shadow
 *      copies below: ordered if at least 1/16 of the word ids of the launch are occurrences of
 *      its 16 most frequent words, or at least 1/48 of its most frequent word (counted on a
 *      sample of the launch's ids, whatever the numbering of the vocabulary); launches without
 *      frequent words (after the reference caller's subsampling, Word2Vec.scala:221-225) keep
 *      the throughput kernels.  A forced w2v_set_hot_update_mode also keeps them.
 *   0  never;  1  always. */
int w2v_set_ordered_mode(int mode);
int w2v_get_ordered_mode(void);
/* Which form the calling thread's most recent update call (any of the operators above) took: 1
 * the ordered form, 0 the throughput kernels, -1 if the thread has made no update call yet (or
 * the counts could not be read).  Waits for the thread's launch stream and reads back the counts
 * that the kernels of that launch looked at; for logs and benchmarks, not for a training loop.
 * No counterpart in the reference. */
int w2v_last_launch_form(void);
/* Number of wavefronts (workers) the ordered form of word2vecPos and of word2vecNeg / NegFilt
 * spreads a launch over; 0 = the library's own numbers (the default).  Fewer workers follow the
 * sequential order more closely and take longer; w2v_set_max_workgroups bounds them as well. */
int w2v_set_ordered_workers(int pos_workers, int neg_workers);
/* In the ordered form the columns of the 16 most frequent words are kept, for the length of a
 * launch, as `copies` x `twins` delta slots next to the (then unchanged) table column: a writer
 * adds to the `twins` slots of one copy, a reader sums one twin of every copy, so no reader misses
 * an update and one cache line takes 1/copies of the adds and 1/twins of the reads.  copies <= 8,
 * copies * twins <= 32; copies = 0: read and update the table columns in place.  Default 2 x 2.
 * The 16 columns are those of ids 0..15: the slots pay when ids are frequency ranks. */
int w2v_set_ordered_copies(int copies, int twins);

/* How the update operators treat the few most frequent words (ids 0..15), whose columns would
 * otherwise serialise the float atomics of the whole device.  No counterpart in the reference.
 *   0  exact: their atomics are spread over shadow copies and every reader sums the copies;
 *   1  combining: a copy is moved into the table on every 8th write to it, and readers read
 *      neither the copies nor the table column but a per-XCD read copy of the column that every
 *      such move refreshes; this hides fewer than 8 updates per copy (a couple of hundred of the
 *      most frequent word) from readers for a few microseconds; about 20 % faster than 0 on a
 *      raw Zipf stream;
 *   2  off: no shadow copies, every column is read and updated in place;
 *  -1  (default) decided per launch and per table on the device: no shadow copies for a table
 *      unless at least 1/16 of the word ids read from it are occurrences of the launch's 16 most
 *      frequent words, or at least 1/48 of its most frequent word (neither holds after
 *      frequent-word subsampling; the second holds for negatives drawn
 *      with the reference's closed form, Word2Vec.scala:349-358); otherwise combining for launches
 *      with at least 2048 wavefronts in flight, where that many updates are invisible to each
 *      other anyway, and exact for smaller ones. */
int w2v_set_hot_update_mode(int mode);
int w2v_get_hot_update_mode(void);

/* How word2vecNeg / word2vecNegFilt update the columns of words that are rare within one call.
 * No counterpart in the reference's GPU path, which uses atomicAdd throughout
 * (jni/src/DNN127.cu:652-661); its CPU path updates every column with a plain read-modify-write from
 * all threads (jni/src/BIDMach_CPUMACH.c:239-254).
 *   0  every update is a float atomic;
 *  -1, 1  (default) the call first counts, on the device, how often each word occurs in it; a word
 *      with so few occurrences that fewer than 1/8 of an update of it is in flight at any time, on
 *      average, is updated with a plain read-modify-write (bit-identical to the atomic update
 *      unless two updates of that column do overlap, in which case one of them is lost, as on the
 *      reference's CPU path).  Frequent words, and every word of a small call, stay atomic.  This
 *      takes about a third of the load off the float-atomic units, which bound the pass.
 *   n >= 2  (tests, experiments) words with at most min(n, 64) occurrences in the call are treated
 *      that way whatever the size of the call. */
int w2v_set_rare_update_mode(int mode);
int w2v_get_rare_update_mode(void);

/* Limits of the tuned kernels: largest nrows (1280) and largest nwb (64).  The four single-table
 * fp32 operators (and word2vecNegFilt, the ...F64, ...Async and ...NoAlloc forms) take any shape:
 * beyond these limits, and for groups of more than 8 B words whose A columns do not fit on chip
 * (about nwa * ceil(nrows/64) > 300), they run one untuned wave-per-unit kernel, as the
 * reference's CPU path takes any nrows, nwa and nwb (BIDMach_CPUMACH.c:37,206,212); that
 * kernel's only bound is nwa * (nwb + 256) <= 16384 for the update (hipErrorInvalidValue
 * beyond).  The sliced and the bfloat16 operators fail with hipErrorInvalidValue beyond the
 * limits. */
int w2v_max_rows(void);
int w2v_max_nwb(void);

/* Device buffers for hosts that have no HIP binding of their own (the reference's host owns its
 * buffers through JCuda; Word2Vec.scala:373 passes their raw pointers). */
int w2v_malloc(void **dev_ptr, size_t bytes);
int w2v_free(void *dev_ptr);
int w2v_memcpy_h2d(void *dev_dst, const void *host_src, size_t bytes);
int w2v_memcpy_d2h(void *host_dst, const void *dev_src, size_t bytes);
int w2v_memset(void *dev_ptr, int value, size_t bytes);

/* Minibatch preprocessing on the device: the step before the operators, what
 * Word2Vec.wordMats does (Word2Vec.scala:214-364; its GPU branch :241-270).  No counterpart in
 * the reference's native library (there it is a chain of BIDMat matrix operations).
 *   mats        device, the 2 x n IMat of the data source, column-major: mats[2*i] word id,
 *               mats[2*i+1] sentence id of token i (swapped when iflip != 0)
 *   wsample_lnv wsample * ln(vocabSize) (Word2Vec.scala:150); wexpt the negative-sampling
 *               exponent (0.75)
 *   seed, call  key of the counter-based random generator; pass a new `call` for every minibatch
 *   words, lb, ub   device int[n] outputs: the W, LB, UB arguments of word2vecPos
 *   negs        device int[nneg * G] output (capacity nneg * ceil(2*nskip*n / nreuse)): WA
 *   ctx         device int[2*nskip*n] output; its first nreuse*G entries are WB
 *   counts_dev  device int[2]: {number of valid pairs, G}; counts_host (may be NULL) gets a copy
 * Blocking (it reads the pair count back to size the rest of the work). */
int w2v_wordmats(int n, const int *mats, int iflip, int vocab, int nskip, int nneg, int nreuse,
                 float wsample_lnv, float wexpt, unsigned long long seed, unsigned call,
                 int *words, int *lb, int *ub, int *negs, int *ctx, int *counts_dev,
                 int *counts_host);

/* Event-pair timers on the calling thread's launch stream. */
int w2v_timer_create(void **timer);
int w2v_timer_destroy(void *timer);
int w2v_timer_start(void *timer);
int w2v_timer_stop(void *timer);
int w2v_timer_elapsed_ms(void *timer, float *ms); /* waits for the stop event */

/* Text of an error code returned by any function above. */
const char *w2v_error_string(int err);

/* LZ4 block codec on HOST memory, for the reference's on-disk files either side of the path:
 * model checkpoints `modelmat%02d.lz4` (Model.scala:259-262, :284-292) and `.imat.lz4` word files.
 * It stands in for the codec BIDMat reaches through lz4-java (both out of the reference tree) and
 * implements the published LZ4 block format; the stream framing is done by the caller.
 * compress/decompress return the number of bytes written, or -1 (output too small, or malformed
 * input, or more than 2^31 - 1 bytes to compress); w2v_lz4_compress_bound(n) bytes of output always
 * suffice to compress n bytes. */
size_t w2v_lz4_compress_bound(size_t n);
long long w2v_lz4_compress(const void *src, size_t n, void *dst, size_t capacity);
long long w2v_lz4_decompress(const void *src, size_t n, void *dst, size_t capacity);

#ifdef __cplusplus
}
#endif

#endif /* BIDMACH_W2V_H_ */
