;;;; hip.lisp -- one MI355X (gfx950) from Lisp: libillatio_hip.so through SBCL's
;;;; alien interface, standing where src/cuda.lisp stands for NVIDIA GPUs.
;;;
;;; UNTESTED: no Lisp exists in the image this repository is built in.  Every
;;; call below is made, with the same arguments, by illatio_amd/hip.py (ctypes),
;;; which the GPU tests go through; this file says the same thing in the
;;; language of the host it is for.
;;;
;;; What it keeps: the names and lambda lists that cuda-dense.lisp and
;;; cuda-ds4f*.lisp call (OPEN-CUDA, CUDA-ALLOC, CUDA-UPLOAD, LAUNCH, ...; the
;;; CUDEV and DBUF structures with the slots those files read), so that loading
;;; this file instead of cuda.lisp changes nothing above it.  What differs
;;; underneath: one library of ours instead of libcuda + NVRTC; no compiling at
;;; OPEN-CUDA (the gfx950 code object is part of the library); LAUNCH hands the
;;; kernel's NAME and the 8-byte-slot argument block to ilt_launch, which
;;; chooses grid and block for 64-lane waves itself (the caller's are read only
;;; where they carry a count: tokens, rows or experts).

(in-package #:illatio)

(defvar *hip-loaded* nil)

(defparameter *hip-library*
  (or (uiop:getenv "ILLATIO_HIP_LIB") "libillatio_hip.so")
  "The shared library: a path, or a name the loader finds.")

(defun load-hip-library ()
  (unless *hip-loaded*
    (sb-alien:load-shared-object *hip-library* :dont-save t)
    (setf *hip-loaded* t)))

;;; The library does no host arithmetic that can trap, but the HIP runtime
;;; under it expects C's floating-point environment as the CUDA driver does.
(defmacro with-cuda (&body body)
  `(sb-int:with-float-traps-masked (:overflow :invalid :inexact :divide-by-zero :underflow)
     ,@body))

(defun hip-error-string (code)
  (or (sb-alien:alien-funcall
       (sb-alien:extern-alien "ilt_error_string" (function sb-alien:c-string sb-alien:int))
       code)
      (format nil "error ~D" code)))

(defmacro ilt (name &rest args)
  "Call the library's NAME with ARGS, each (alien-type value); signal unless
   it returns 0.  Every entry point returns an int, 0 for success."
  (let ((r (gensym)))
    `(let ((,r (sb-alien:alien-funcall
                (sb-alien:extern-alien ,name (function sb-alien:int ,@(mapcar #'first args)))
                ,@(mapcar #'second args))))
       (unless (zerop ,r) (error "HIP: ~A: ~A" ,name (hip-error-string ,r)))
       ,r)))

(defmacro with-out ((&rest vars) &body body)
  "Each VAR a fresh 64-bit out-parameter cell; BODY passes (out-ptr VAR)."
  `(sb-alien:with-alien ,(mapcar (lambda (v) `(,v sb-alien:unsigned-long 0)) vars)
     ,@body))

(defmacro out-ptr (var) `(sb-alien:alien-sap (sb-alien:addr ,var)))

;;; --- devices ------------------------------------------------------------------

(defstruct (cudev (:constructor %make-cudev))
  (index 0 :type fixnum)
  name
  ctx                                   ; unused here: the runtime's device is set by index
  stream
  module                                ; unused here: the kernels are inside the library
  arch                                  ; reported as 90: the callers' (>= arch 80) tests take the matrix-core paths
  (total-memory 0)
  (max-shared 65536)                    ; LDS bytes a workgroup may use (the library opts in by itself)
  (numa-node -1)
  (compute-units 0)
  (wave-size 64)
  ;; LAUNCH's argument block: 64 values of 8 bytes, then 64 pointers to them
  (params (sb-sys:int-sap 0)))

(defvar *cuda-devices* (make-hash-table) "Index -> open CUDEV.")

(defun cuda-device-count ()
  (load-hip-library)
  (with-cuda
    (ilt "ilt_init")
    (sb-alien:with-alien ((n sb-alien:int 0))
      (ilt "ilt_device_count" ((* sb-alien:int) (sb-alien:addr n)))
      n)))

(defun cuda-current (dev)
  "Make DEV the calling thread's device."
  (ilt "ilt_set_device" (sb-alien:int (cudev-index dev))))

(defun open-cuda (&optional (index 0))
  "Device INDEX, opened once: its description and a stream."
  (or (gethash index *cuda-devices*)
      (setf (gethash index *cuda-devices*) (open-hip-1 index))))

;; struct ilt_device_info (include/illatio_hip.h): char name[256]; int arch;
;; uint64 total_memory (at 264); int max_shared, numa_node, compute_units, wave_size (at 272..).
(defconstant +device-info-bytes+ 288)

(defun open-hip-1 (index)
  (load-hip-library)
  (with-cuda
    (ilt "ilt_init")
    (let ((info (make-array +device-info-bytes+ :element-type '(unsigned-byte 8) :initial-element 0)))
      (sb-sys:with-pinned-objects (info)
        (let ((sap (sb-sys:vector-sap info)))
          (ilt "ilt_device_get_info" (sb-alien:int index) (sb-sys:system-area-pointer sap))
          (ilt "ilt_set_device" (sb-alien:int index))
          (with-out (stream)
            (ilt "ilt_stream_create" (sb-sys:system-area-pointer (out-ptr stream)) (sb-alien:unsigned 0))
            (%make-cudev :index index
                         :name (sb-ext:octets-to-string (subseq info 0 (or (position 0 info :end 256) 256)))
                         :arch (sb-sys:signed-sap-ref-32 sap 256)
                         :total-memory (sb-sys:sap-ref-64 sap 264)
                         :max-shared (sb-sys:signed-sap-ref-32 sap 272)
                         :numa-node (sb-sys:signed-sap-ref-32 sap 276)
                         :compute-units (sb-sys:signed-sap-ref-32 sap 280)
                         :wave-size (sb-sys:signed-sap-ref-32 sap 284)
                         :stream (sb-sys:int-sap stream)
                         :params (sb-sys:int-sap (%mmap-anon (* 2 64 8))))))))))

;;; --- memory -------------------------------------------------------------------

(defstruct (dbuf (:constructor %make-dbuf))
  (ptr 0 :type (unsigned-byte 64)) (bytes 0 :type (unsigned-byte 62)) dev)

(defvar *cuda-alloc-hook* nil
  "A function called with each new DBUF, or NIL.")

(defun stream-handle (dev) (sb-sys:sap-int (cudev-stream dev)))

(defun cuda-alloc (dev bytes &key (zero t))
  "BYTES of DEV's memory (zeroed unless ZERO is NIL)."
  (with-cuda
    (cuda-current dev)
    (with-out (p)
      (ilt "ilt_malloc" (sb-sys:system-area-pointer (out-ptr p)) (sb-alien:unsigned-long (max bytes 256)))
      (let ((b (%make-dbuf :ptr p :bytes bytes :dev dev)))
        (when zero (cuda-zero b))
        (when *cuda-alloc-hook* (funcall *cuda-alloc-hook* b))
        b))))

(defun cuda-realloc (b)
  "Device memory again for B, freed: a new address in the same DBUF."
  (assert (zerop (dbuf-ptr b)))
  (with-cuda
    (cuda-current (dbuf-dev b))
    (with-out (p)
      (ilt "ilt_malloc" (sb-sys:system-area-pointer (out-ptr p)) (sb-alien:unsigned-long (max (dbuf-bytes b) 256)))
      (setf (dbuf-ptr b) p)))
  b)

(defun cuda-free (b)
  (when (and b (plusp (dbuf-ptr b)))
    (with-cuda
      (cuda-current (dbuf-dev b))
      (ilt "ilt_free" (sb-alien:unsigned-long (dbuf-ptr b))))
    (setf (dbuf-ptr b) 0))
  nil)

(defun cuda-zero (b)
  (with-cuda
    (ilt "ilt_memset_async" (sb-alien:unsigned-long (dbuf-ptr b)) (sb-alien:int 0)
         (sb-alien:unsigned-long (dbuf-bytes b)) (sb-alien:unsigned-long (stream-handle (dbuf-dev b)))))
  b)

(defun cuda-mem-info (dev)
  "(VALUES free total) bytes on DEV."
  (with-cuda
    (cuda-current dev)
    (with-out (f tot)
      (ilt "ilt_mem_info" (sb-sys:system-area-pointer (out-ptr f)) (sb-sys:system-area-pointer (out-ptr tot)))
      (values f tot))))

(defun cuda-sync (dev)
  (with-cuda (ilt "ilt_stream_sync" (sb-alien:unsigned-long (stream-handle dev)))))

(defun cuda-upload (b sap bytes &optional (offset 0))
  "BYTES at host address SAP into B at OFFSET; returns when the copy is made."
  (with-cuda
    (let ((dev (dbuf-dev b)))
      (ilt "ilt_memcpy_htod_async" (sb-alien:unsigned-long (+ (dbuf-ptr b) offset))
           (sb-sys:system-area-pointer sap) (sb-alien:unsigned-long bytes)
           (sb-alien:unsigned-long (stream-handle dev)))
      (cuda-sync dev))))

(defun cuda-upload-vector (b v &optional (offset 0))
  "The specialized vector V's bytes into B at OFFSET."
  (let ((bytes (* (length v) (etypecase v
                               ((simple-array single-float (*)) 4) ((simple-array (signed-byte 32) (*)) 4)
                               ((simple-array (unsigned-byte 32) (*)) 4)
                               ((simple-array (unsigned-byte 8) (*)) 1) ((simple-array (signed-byte 8) (*)) 1)))))
    (sb-sys:with-pinned-objects (v)
      (cuda-upload b (sb-sys:vector-sap v) bytes offset))
    b))

(defun cuda-download (b sap bytes &optional (offset 0))
  "BYTES of B at OFFSET to host address SAP, after the work queued before it."
  (with-cuda
    (let ((dev (dbuf-dev b)))
      (ilt "ilt_memcpy_dtoh_async" (sb-sys:system-area-pointer sap)
           (sb-alien:unsigned-long (+ (dbuf-ptr b) offset)) (sb-alien:unsigned-long bytes)
           (sb-alien:unsigned-long (stream-handle dev)))
      (cuda-sync dev))))

(defun cuda-floats (b n &optional (start 0))
  "Floats START..START+N-1 of B, as a vector."
  (let ((v (make-array n :element-type 'single-float)))
    (sb-sys:with-pinned-objects (v)
      (cuda-download b (sb-sys:vector-sap v) (* 4 n) (* 4 start)))
    v))

;;; --- launching ----------------------------------------------------------------

(defun launch (dev kernel grid block args &key (shared 0))
  "Queue KERNEL on DEV's stream.  ARGS in the kernel's order: DBUFs or
   (DBUF . byte-offset) for pointers, NIL for a null pointer, integers for
   ints, single-floats for floats, (:I64 n) for a long long -- each in an
   8-byte slot, the block cuLaunchKernel took.  GRID and BLOCK are passed on;
   the library reads them only where a count lives in them (d4_route: tokens
   = grid x; embed_*: rows = grid x; the expert kernels: experts = grid z;
   rmsnorm_q8, qk_rope, attn_rows: rows or tokens = grid y) and derives the
   launch shape from the kernel's arguments.  SHARED is ignored: the library
   asks for the LDS its kernels need."
  (let ((pv (cudev-params dev)))
    (loop for a in args for i from 0
          for slot = (sb-sys:sap+ pv (* 8 i))
          do (etypecase a
               (null (setf (sb-sys:sap-ref-64 slot 0) 0))
               (dbuf (setf (sb-sys:sap-ref-64 slot 0) (dbuf-ptr a)))
               ((cons dbuf integer) (setf (sb-sys:sap-ref-64 slot 0) (+ (dbuf-ptr (car a)) (cdr a))))
               ((cons (eql :i64)) (setf (sb-sys:sap-ref-64 slot 0) (ldb (byte 64 0) (second a))))
               (integer (setf (sb-sys:sap-ref-64 slot 0) (ldb (byte 32 0) a)))
               (single-float (setf (sb-sys:sap-ref-64 slot 0) 0
                                   (sb-sys:sap-ref-single slot 0) a)))
             (setf (sb-sys:sap-ref-sap pv (* 8 (+ 64 i))) slot))
    (flet ((dim (x k) (let ((l (if (listp x) x (list x)))) (or (nth k l) 1))))
      (with-cuda
        (cuda-current dev)
        (ilt "ilt_launch" (sb-alien:c-string kernel)
             (sb-alien:unsigned (dim grid 0)) (sb-alien:unsigned (dim grid 1)) (sb-alien:unsigned (dim grid 2))
             (sb-alien:unsigned (dim block 0)) (sb-alien:unsigned (dim block 1)) (sb-alien:unsigned (dim block 2))
             (sb-alien:unsigned shared) (sb-alien:unsigned-long (stream-handle dev))
             (sb-sys:system-area-pointer (sb-sys:sap+ pv (* 8 64))))))))

;;; --- pinned host memory, more streams, events ----------------------------------

(defun cuda-host-alloc (bytes &key mapped)
  "BYTES of pinned host memory (portable): its SAP.  MAPPED: kernels may read
   it where it lies, at the same address -- an expert left in host memory is
   read through this way (its address goes into the table of slots)."
  (with-cuda
    (with-out (p)
      (ilt "ilt_host_alloc" (sb-sys:system-area-pointer (out-ptr p)) (sb-alien:unsigned-long (max bytes 64))
           (sb-alien:unsigned (if mapped 3 1)))
      (sb-sys:int-sap p))))

(defun cuda-host-free (sap)
  (with-cuda (ilt "ilt_host_free" (sb-alien:unsigned-long (sb-sys:sap-int sap)))))

(defun cuda-host-register (sap bytes)
  "Refused by the library (error 801): the MI355X hosts this was built on do
   not pin memory that already exists.  Callers that stream experts from a
   file read into CUDA-HOST-ALLOC memory instead of registering the mapping."
  (with-cuda
    (ilt "ilt_host_register" (sb-sys:system-area-pointer sap) (sb-alien:unsigned-long bytes)
         (sb-alien:unsigned 3)))
  sap)

(defun cuda-host-unregister (sap)
  (with-cuda (ilt "ilt_host_unregister" (sb-sys:system-area-pointer sap))))

(defun cuda-stream-create (dev)
  "A new stream on DEV that doesn't wait for its default stream."
  (with-cuda
    (cuda-current dev)
    (with-out (s)
      (ilt "ilt_stream_create" (sb-sys:system-area-pointer (out-ptr s)) (sb-alien:unsigned 1))
      (sb-sys:int-sap s))))

(defun cuda-event-create (dev)
  (with-cuda
    (cuda-current dev)
    (with-out (e)
      (ilt "ilt_event_create" (sb-sys:system-area-pointer (out-ptr e)) (sb-alien:unsigned 2)) ; no timing
      (sb-sys:int-sap e))))

(defun cuda-event-destroy (event)
  (with-cuda (ilt "ilt_event_destroy" (sb-alien:unsigned-long (sb-sys:sap-int event)))))

(defun cuda-event-record (event stream)
  (with-cuda (ilt "ilt_event_record" (sb-alien:unsigned-long (sb-sys:sap-int event))
                  (sb-alien:unsigned-long (sb-sys:sap-int stream)))))

(defun cuda-stream-wait (stream event)
  "STREAM's later work waits for EVENT."
  (with-cuda (ilt "ilt_stream_wait_event" (sb-alien:unsigned-long (sb-sys:sap-int stream))
                  (sb-alien:unsigned-long (sb-sys:sap-int event)))))

(defun cuda-stream-sync (stream)
  (with-cuda (ilt "ilt_stream_sync" (sb-alien:unsigned-long (sb-sys:sap-int stream)))))

(defun cuda-copy-in (b offset sap bytes &optional (stream (cudev-stream (dbuf-dev b))))
  "BYTES at host SAP into B at OFFSET, queued on STREAM (asynchronous when SAP is pinned)."
  (with-cuda
    (ilt "ilt_memcpy_htod_async" (sb-alien:unsigned-long (+ (dbuf-ptr b) offset))
         (sb-sys:system-area-pointer sap) (sb-alien:unsigned-long bytes)
         (sb-alien:unsigned-long (sb-sys:sap-int stream)))))

(defun cuda-copy-dd (dst dst-offset src src-offset bytes)
  (with-cuda
    (ilt "ilt_memcpy_dtod_async" (sb-alien:unsigned-long (+ (dbuf-ptr dst) dst-offset))
         (sb-alien:unsigned-long (+ (dbuf-ptr src) src-offset)) (sb-alien:unsigned-long bytes)
         (sb-alien:unsigned-long (stream-handle (dbuf-dev dst))))))

(defun cuda-copy-out (sap b offset bytes)
  "BYTES of B at OFFSET to host SAP, queued on B's device's stream (no wait)."
  (with-cuda
    (ilt "ilt_memcpy_dtoh_async" (sb-sys:system-area-pointer sap)
         (sb-alien:unsigned-long (+ (dbuf-ptr b) offset)) (sb-alien:unsigned-long bytes)
         (sb-alien:unsigned-long (stream-handle (dbuf-dev b))))))

(defun cuda-event-done-p (event)
  "Whether the work before EVENT's last record has finished."
  (let ((r (with-cuda (sb-alien:alien-funcall
                       (sb-alien:extern-alien "ilt_event_query" (function sb-alien:int sb-alien:unsigned-long))
                       (sb-sys:sap-int event)))))
    (cond ((zerop r) t)
          ((= r 600) nil)                   ; ILT_NOT_READY, the value CUDA gives
          (t (error "HIP: ilt_event_query: ~A" (hip-error-string r))))))

;;; --- what the hosts above call beyond LAUNCH -------------------------------------
;;; Typed entry points whose arguments do not fit the slot block (a struct, or
;;; a caller's workspace); see include/illatio_hip.h for each.

(defun hip-d4-ffn-step-workspace (nu d ff)
  "Bytes of workspace ilt_d4_ffn_step wants for NU slots of a D x FF expert."
  (sb-alien:alien-funcall
   (sb-alien:extern-alien "ilt_d4_ffn_step_workspace"
                          (function sb-alien:unsigned-long sb-alien:int sb-alien:int sb-alien:int))
   nu d ff))

(defun hip-d4-ffn-step (dev ws weights-sap ne nu d ff scale clamp logits bias x moe)
  "One token's FFN past the router in one call (four launches, the routing on
   the device): what DK-FFN-HEAD's shared expert, the logits' copy-out, the
   wait, D4-ROUTE and DK-FFN-TAIL do together (cuda-ds4f.lisp:908-1013).
   WS a DBUF of HIP-D4-FFN-STEP-WORKSPACE bytes; WEIGHTS-SAP an
   ilt_ffn_step_weights in foreign memory (the slot table's address, the
   gate's byte size, the shared expert's six arrays)."
  (with-cuda
    (cuda-current dev)
    (ilt "ilt_d4_ffn_step" (sb-alien:unsigned-long (stream-handle dev))
         (sb-alien:unsigned-long (dbuf-ptr ws)) (sb-alien:unsigned-long (dbuf-bytes ws))
         (sb-alien:int ne) (sb-alien:int nu) (sb-alien:int d) (sb-alien:int ff)
         (sb-alien:single-float scale) (sb-alien:single-float clamp)
         (sb-sys:system-area-pointer weights-sap)
         (sb-alien:unsigned-long (dbuf-ptr logits)) (sb-alien:unsigned-long (if bias (dbuf-ptr bias) 0))
         (sb-alien:unsigned-long (dbuf-ptr x)) (sb-alien:unsigned-long (dbuf-ptr moe)))))

(defun hip-dense-decode (dev model-sap token-buf pos want-logits)
  "One token of the dense decoder queued by one call (CUDA-FORWARD-N for one
   token, cuda-dense.lisp:380-432): MODEL-SAP an ilt_dense_model in foreign
   memory, TOKEN-BUF a DBUF holding the token's id."
  (with-cuda
    (cuda-current dev)
    (ilt "ilt_dense_decode" (sb-alien:unsigned-long (stream-handle dev))
         (sb-sys:system-area-pointer model-sap) (sb-alien:unsigned-long (dbuf-ptr token-buf))
         (sb-alien:int pos) (sb-alien:int (if want-logits 1 0)))))
