// JNI glue between edu.berkeley.bid.CUMACH's word2vec natives and the C ABI of the HIP library.
//
// It answers the part of the reference's jni/src/BIDMach_CUMACH.cpp that binds these natives
// (:434-493, with the field-id set-up of JNI_OnLoad, :12-30) for the declarations in
// src/main/java/edu/berkeley/bid/CUMACH.java:90,92,94,96,98.  A jcuda.Pointer carries a native
// address and a byte offset (jni/src/PointerUtils.cpp:55-91; getPointer, :353-363); the device
// address handed to the library is their sum, whatever allocator the address came from.
//
// Built by jni/Makefile into libbidmachcuda-linux-x86_64.so, the artefact name the Java side
// loads (CUMACH.java:9, jni/src/Makefile:20-21), only where a JDK's jni.h is found.  The C
// functions return 0 or a hipError_t value; the Scala caller throws on non-zero as it does today
// (Word2Vec.scala:374,393,478,512).
#include <jni.h>

#include "../include/bidmach_w2v.h"

namespace {

jfieldID g_native_pointer = nullptr;
jfieldID g_byte_offset = nullptr;

template <typename T>
T* device_ptr(JNIEnv* env, jobject pointer) {
  if (pointer == nullptr) return nullptr;
  const jlong base = env->GetLongField(pointer, g_native_pointer);
  const jlong offset = env->GetLongField(pointer, g_byte_offset);
  return reinterpret_cast<T*>(static_cast<intptr_t>(base + offset));
}

}  // namespace

extern "C" {

JNIEXPORT jint JNICALL JNI_OnLoad(JavaVM* vm, void*) {
  JNIEnv* env = nullptr;
  if (vm->GetEnv(reinterpret_cast<void**>(&env), JNI_VERSION_1_4) != JNI_OK) return JNI_ERR;
  jclass native_pointer_object = env->FindClass("jcuda/NativePointerObject");
  jclass pointer = env->FindClass("jcuda/Pointer");
  if (native_pointer_object == nullptr || pointer == nullptr) return JNI_ERR;
  g_native_pointer = env->GetFieldID(native_pointer_object, "nativePointer", "J");
  g_byte_offset = env->GetFieldID(pointer, "byteOffset", "J");
  if (g_native_pointer == nullptr || g_byte_offset == nullptr) return JNI_ERR;
  return JNI_VERSION_1_4;
}

JNIEXPORT jint JNICALL Java_edu_berkeley_bid_CUMACH_word2vecPos(
    JNIEnv* env, jobject, jint nrows, jint ncols, jint shift, jobject jW, jobject jLB, jobject jUB,
    jobject jA, jobject jB, jfloat lrate, jfloat vexp) {
  return word2vecPos(nrows, ncols, shift, device_ptr<int>(env, jW), device_ptr<int>(env, jLB),
                     device_ptr<int>(env, jUB), device_ptr<float>(env, jA),
                     device_ptr<float>(env, jB), lrate, vexp);
}

JNIEXPORT jint JNICALL Java_edu_berkeley_bid_CUMACH_word2vecNeg(
    JNIEnv* env, jobject, jint nrows, jint ncols, jint nwa, jint nwb, jobject jWA, jobject jWB,
    jobject jA, jobject jB, jfloat lrate, jfloat vexp) {
  return word2vecNeg(nrows, ncols, nwa, nwb, device_ptr<int>(env, jWA), device_ptr<int>(env, jWB),
                     device_ptr<float>(env, jA), device_ptr<float>(env, jB), lrate, vexp);
}

JNIEXPORT jint JNICALL Java_edu_berkeley_bid_CUMACH_word2vecNegFilt(
    JNIEnv* env, jobject, jint nrows, jint ncols, jint nwords, jint nwa, jint nwb, jobject jWA,
    jobject jWB, jobject jA, jobject jB, jfloat lrate, jfloat vexp) {
  return word2vecNegFilt(nrows, ncols, nwords, nwa, nwb, device_ptr<int>(env, jWA),
                         device_ptr<int>(env, jWB), device_ptr<float>(env, jA),
                         device_ptr<float>(env, jB), lrate, vexp);
}

JNIEXPORT jint JNICALL Java_edu_berkeley_bid_CUMACH_word2vecEvalPos(
    JNIEnv* env, jobject, jint nrows, jint ncols, jint shift, jobject jW, jobject jLB, jobject jUB,
    jobject jA, jobject jB, jobject jRetval) {
  return word2vecEvalPos(nrows, ncols, shift, device_ptr<int>(env, jW), device_ptr<int>(env, jLB),
                         device_ptr<int>(env, jUB), device_ptr<float>(env, jA),
                         device_ptr<float>(env, jB), device_ptr<float>(env, jRetval));
}

JNIEXPORT jint JNICALL Java_edu_berkeley_bid_CUMACH_word2vecEvalNeg(
    JNIEnv* env, jobject, jint nrows, jint ncols, jint nwa, jint nwb, jobject jWA, jobject jWB,
    jobject jA, jobject jB, jobject jRetval) {
  return word2vecEvalNeg(nrows, ncols, nwa, nwb, device_ptr<int>(env, jWA),
                         device_ptr<int>(env, jWB), device_ptr<float>(env, jA),
                         device_ptr<float>(env, jB), device_ptr<float>(env, jRetval));
}

// A JVM worker thread that has called the operators holds device scratch memory of its own;
// call this before such a thread ends (no counterpart in the reference, whose kernels keep no
// state).  Bind it as `public static native int w2vReleaseThread();` in CUMACH.java.
JNIEXPORT jint JNICALL Java_edu_berkeley_bid_CUMACH_w2vReleaseThread(JNIEnv*, jobject) {
  return w2v_release_thread();
}

}  // extern "C"
