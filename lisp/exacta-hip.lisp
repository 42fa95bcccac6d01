;;;; exacta-hip.lisp -- the SBCL side of libexacta_hip.so: Exacta's PROVE with its data-parallel loops on an
;;;; MI355X (gfx950).
;;;;
;;;; Load after the "exacta" system.  The host keeps PROVE / VERIFY / CHECK-FINAL, the s-expression statements,
;;;; the transcript and the proof format (src/sumcheck.lisp:131-172, 512-571); what moves to the device is the
;;;; body of the round loop: MAKE-TABLE's upload (:531), the round kernel call (:556), FOLD-FLAT-TABLE (:562) and
;;;; the read-back of finals and folded tables (:564-571) -- plus, with PROVE/HIP's :CHAINED mode, SEND and
;;;; CHALLENGE of the rounds on the device's copy of the transcript's hash state, replayed here afterwards.
;;;; Calling convention (the reference's own notes on SBCL -> C calls): inline DEFINE-ALIEN-ROUTINEs, specialised
;;;; (unsigned-byte 32) vectors passed as SB-SYS:VECTOR-SAP inside SB-SYS:WITH-PINNED-OBJECTS, never
;;;; WITHOUT-GCING, one call per whole array.  The library never calls back into Lisp and never continues past
;;;; a rejection: every entry point returns a status, mapped to the reference's conditions by CHECK.
;;;;
;;;; No Lisp implementation exists where this library is built and tested, so this file has not been run
;;;; there; the same C entry points are exercised by the library's tests through its C++ host mirror.

(defpackage #:exacta.hip
  (:use #:cl #:sb-alien #:exacta.util #:exacta.conditions #:exacta.field #:exacta.forms #:exacta.blake3
        #:exacta.transcript)
  (:import-from #:exacta.sumcheck #:header #:statement-degree)
  (:export #:*library* #:load-library #:init #:shutdown #:device-error
           #:upload-table #:free-table #:download-table
           #:compile-statement #:free-statement
           #:begin-session #:session-round #:session-fold #:session-run #:finish-session
           #:prove/hip
           #:rs-encode/hip #:merkle-commit/hip #:rs-fold/hip #:gkr-reduce-layer/hip
           #:combine-columns/hip #:dot-pairs/hip #:fold-table/hip))

(in-package #:exacta.hip)

;;; ------------------------------------------------------------------ loading

(defvar *library* "libexacta_hip.so"
  "Path of the shared library (built by `make -C sable_amd/csrc`).")

(defun load-library (&optional (path *library*))
  (load-shared-object path)
  path)

;;; ------------------------------------------------------------------ status codes -> conditions
;;; include/exacta_hip.h: EXH_OK 0, EXH_E_PARAM -1, EXH_E_DIVZERO -2, EXH_E_SHAPE -3, EXH_E_EXHAUSTED -4,
;;; EXH_E_REJECT -5, EXH_E_MALFORMED -6, EXH_E_DEVICE -7, EXH_E_NOMEM -8, named after src/conditions.lisp.

(define-condition device-error (exacta-error)
  ((status :initarg :status :reader device-error-status)
   (message :initarg :message :reader device-error-message))
  (:report (lambda (c stream)
             (format stream "libexacta_hip: ~A (status ~D)" (device-error-message c) (device-error-status c))))
  (:documentation "No usable gfx950 device, a HIP call failed, or device memory ran out."))

(declaim (inline %last-error))
(define-alien-routine ("exh_last_error" %last-error) c-string)

(defun check (status)
  "A non-zero STATUS becomes the condition of the reference's class it is named after
(src/conditions.lisp:38-120); the library's message rides along as the detail."
  (unless (zerop status)
    (let ((message (or (%last-error) "")))
      (case status
        (-1 (error 'invalid-parameter :name :libexacta-hip :value message :expected "see the message"))
        (-2 (error 'field-division-by-zero))
        (-3 (error 'message-shape-error :index nil :expected :see-detail :actual message :detail message))
        (-4 (error 'transcript-exhausted :index nil :detail message))
        (-5 (error 'verification-failure :check :libexacta-hip :detail message))
        (-6 (error 'malformed-proof :reason :truncated :detail message))
        (t (error 'device-error :status status :message message)))))
  status)

;;; ------------------------------------------------------------------ the alien routines
;;; One per entry point of include/exacta_hip.h that the sumcheck, GKR, Reed-Solomon and Merkle paths bind.

(declaim (inline %init %shutdown %synchronize
                 %table-upload %table-alloc %table-download %table-free
                 %stmt-compile %stmt-degree %stmt-free %stmt-generate
                 %sumcheck-begin %sumcheck-round %sumcheck-fold %sumcheck-run %sumcheck-finish
                 %rs-encode %merkle-commit %rs-fold %gkr-reduce-layer
                 %combine-columns %dot-pairs %fold-table %eq-table-device))

(define-alien-routine ("exh_init" %init) int (device int))
(define-alien-routine ("exh_shutdown" %shutdown) void)
(define-alien-routine ("exh_synchronize" %synchronize) int)

(define-alien-routine ("exh_table_upload" %table-upload) int
  (host system-area-pointer) (n-u32 (unsigned 64)) (stride int) (out (* (unsigned 64))))
(define-alien-routine ("exh_table_alloc" %table-alloc) int
  (n-u32 (unsigned 64)) (stride int) (out (* (unsigned 64))))
(define-alien-routine ("exh_table_download" %table-download) int
  (table (unsigned 64)) (offset-u32 (unsigned 64)) (host system-area-pointer) (n-u32 (unsigned 64)))
(define-alien-routine ("exh_table_free" %table-free) int (table (unsigned 64)))

(define-alien-routine ("exh_stmt_compile" %stmt-compile) int
  (form c-string) (tables (* c-string)) (n-tables int) (constants (* c-string)) (n-constants int)
  (out (* (unsigned 64))))
(define-alien-routine ("exh_stmt_degree" %stmt-degree) int (stmt (unsigned 64)))
(define-alien-routine ("exh_stmt_free" %stmt-free) int (stmt (unsigned 64)))
(define-alien-routine ("exh_stmt_generate" %stmt-generate) int
  (stmt (unsigned 64)) (degree-d int) (degree int) (wait int))

(define-alien-routine ("exh_sumcheck_begin" %sumcheck-begin) int
  (stmt (unsigned 64)) (degree-d int) (n int) (tables (* (unsigned 64))) (n-tables int)
  (eq system-area-pointer) (block-weights system-area-pointer) (k int) (constants system-area-pointer)
  (degree int) (out (* (unsigned 64))))
(define-alien-routine ("exh_sumcheck_round" %sumcheck-round) int
  (session (unsigned 64)) (out-sums system-area-pointer))
(define-alien-routine ("exh_sumcheck_fold" %sumcheck-fold) int
  (session (unsigned 64)) (r system-area-pointer))
(define-alien-routine ("exh_sumcheck_run" %sumcheck-run) int
  (session (unsigned 64)) (cv system-area-pointer) (block system-area-pointer) (used (unsigned 32))
  (counter (unsigned 64)) (out-messages system-area-pointer) (out-challenges system-area-pointer))
(define-alien-routine ("exh_sumcheck_finish" %sumcheck-finish) int
  (session (unsigned 64)) (finals system-area-pointer) (folded (* system-area-pointer)))

(define-alien-routine ("exh_rs_encode" %rs-encode) int
  (messages (unsigned 64)) (ncols int) (c int) (codewords (* (unsigned 64))))
(define-alien-routine ("exh_merkle_commit" %merkle-commit) int
  (codewords (unsigned 64)) (ncols int) (c int) (levels (* (unsigned 64))) (cap system-area-pointer)
  (cap-rows (* (unsigned 64))))
(define-alien-routine ("exh_rs_fold" %rs-fold) int
  (codeword (unsigned 64)) (degree-d int) (m (unsigned 64)) (n-domain int) (level int) (r system-area-pointer)
  (out (* (unsigned 64))))
(define-alien-routine ("exh_gkr_reduce_layer" %gkr-reduce-layer) int
  (p (unsigned 64)) (q (unsigned 64)) (degree-d int) (k int) (m int)
  (out-p (* (unsigned 64))) (out-q (* (unsigned 64))))
(define-alien-routine ("exh_combine_columns" %combine-columns) int
  (columns (unsigned 64)) (ncols int) (len (unsigned 64)) (degree-d int) (coefficients system-area-pointer)
  (out (* (unsigned 64))))
(define-alien-routine ("exh_dot_pairs" %dot-pairs) int
  (e (unsigned 64)) (v (unsigned 64)) (out system-area-pointer))
(define-alien-routine ("exh_fold_table" %fold-table) int
  (table (unsigned 64)) (r system-area-pointer) (out (* (unsigned 64))))
(define-alien-routine ("exh_eq_table_device" %eq-table-device) int
  (degree-d int) (k int) (r system-area-pointer) (out (* (unsigned 64))))

;;; ------------------------------------------------------------------ context

(defun init (&optional (device 0))
  "exh_init: once per process, before anything else."
  (check (%init device)))

(defun shutdown ()
  (%shutdown))

;;; ------------------------------------------------------------------ flat vectors

(defun u32-vector (n)
  (make-array n :element-type '(unsigned-byte 32) :initial-element 0))

(defun flatten-exts (exts d)
  "A sequence of EXTs (or NIL) as one (unsigned-byte 32) vector of D words each, canonical; NIL -> NIL."
  (when exts
    (let* ((exts (coerce exts 'vector))
           (flat (u32-vector (* d (length exts)))))
      (loop for e across exts
            for x from 0
            do (replace flat (if (integerp e) (base->ext e d) e) :start1 (* d x)))
      flat)))

(defmacro with-sap ((sap vector) &body body)
  "Bind SAP to VECTOR's data for the length of BODY (a null pointer when VECTOR is NIL).  The vector is
pinned, not copied, and the collector keeps running (never WITHOUT-GCING)."
  (let ((v (gensym "VECTOR")))
    `(let ((,v ,vector))
       (if ,v
           (sb-sys:with-pinned-objects (,v)
             (let ((,sap (sb-sys:vector-sap ,v))) ,@body))
           (let ((,sap (sb-sys:int-sap 0))) ,@body)))))

;;; ------------------------------------------------------------------ tables (MAKE-TABLE, src/sumcheck.lisp:61-70)

(defun upload-table (values d)
  "VALUES as MAKE-TABLE lays them out -- stride 1 when every value is an integer, else stride D with the
integers lifted -- uploaded once; returns the table's handle and stride.  Values must be canonical
(the library refuses one that is not below p, as ENCODE-PROOF does)."
  (let* ((values (coerce values 'vector))
         (base (every #'integerp values))
         (stride (if base 1 d))
         (flat (if base (coerce-ext values) (flatten-exts values d))))
    (with-alien ((out (unsigned 64)))
      (with-sap (sap flat)
        (check (%table-upload sap (length flat) stride (addr out))))
      (values out stride))))

(defun free-table (handle)
  (check (%table-free handle)))

(defun download-table (handle n-u32 &optional (offset-u32 0))
  (let ((out (u32-vector n-u32)))
    (with-sap (sap out)
      (check (%table-download handle offset-u32 sap n-u32)))
    out))

;;; ------------------------------------------------------------------ statements (COMPILE-FORM / ROUND-KERNEL)

(defun call-with-c-strings (strings function)
  "Call FUNCTION with a foreign array of C strings holding STRINGS (freed afterwards) and their count."
  (let* ((n (length strings))
         (array (make-alien c-string (max n 1))))
    (unwind-protect
         (progn
           (loop for s in strings
                 for i from 0
                 do (setf (deref array i) s))     ; SETF of a C-STRING alien makes a foreign copy
           (funcall function array n))
      (loop for i below n do (free-alien (deref array i)))
      (free-alien array))))

(defun variable-name (symbol)
  "A statement variable as the library spells it: the symbol's name, as FORM-VARIABLES sorts by it."
  (string-downcase (symbol-name symbol)))

(defun compile-statement (statement table-names constant-names)
  "exh_stmt_compile of STATEMENT's printed s-expression with its variables in the order their values will
be passed: the tables (an alist's CARs, as PROVE receives them), then the constants.  The library expands
the form into the reference's canonical sum of monomials (EXPAND, src/forms.lisp:57-78) and picks or
generates the kernels; returns the statement's handle."
  (let ((form (let ((*print-case* :downcase) (*package* (find-package :keyword)))
                (prin1-to-string statement))))
    (with-alien ((out (unsigned 64)))
      (call-with-c-strings
       (mapcar #'variable-name table-names)
       (lambda (tables n-tables)
         (call-with-c-strings
          (mapcar #'variable-name constant-names)
          (lambda (constants n-constants)
            (check (%stmt-compile form tables n-tables constants n-constants (addr out)))))))
      out)))

(defun free-statement (handle)
  (check (%stmt-free handle)))

;;; ------------------------------------------------------------------ one sumcheck, round by round

(defstruct (session (:constructor %make-session))
  handle d n points (tables 0 :type fixnum) (blocks 1 :type fixnum))

(defun begin-session (stmt d n table-handles eq block-weights constant-values degree)
  "exh_sumcheck_begin: TABLE-HANDLES in the statement's table order; EQ a list of N EXTs or NIL;
BLOCK-WEIGHTS K EXTs or NIL; CONSTANT-VALUES EXTs in the statement's constant order."
  (let* ((k (if block-weights (length block-weights) 1))
         (nt (length table-handles))
         (eq-flat (flatten-exts eq d))
         (bw-flat (flatten-exts block-weights d))
         (const-flat (flatten-exts constant-values d))
         (handles (make-alien (unsigned 64) (max nt 1))))
    (unwind-protect
         (with-alien ((out (unsigned 64)))
           (loop for h in table-handles for i from 0 do (setf (deref handles i) h))
           (with-sap (eq-sap eq-flat)
             (with-sap (bw-sap bw-flat)
               (with-sap (const-sap const-flat)
                 (check (%sumcheck-begin stmt d n handles nt eq-sap bw-sap k const-sap degree (addr out))))))
           (%make-session :handle out :d d :n n :points (max degree 1) :tables nt :blocks k))
      (free-alien handles))))

(defun session-round (session)
  "The round kernel call (src/sumcheck.lisp:556): the message's rows at X = 0, 2, 3, ... as a (points D)
field array, ready for SEND."
  (let* ((points (session-points session))
         (d (session-d session))
         (sums (u32-vector (* points d))))
    (with-sap (sap sums)
      (check (%sumcheck-round (session-handle session) sap)))
    (make-array (list points d) :element-type '(unsigned-byte 32) :displaced-to sums)))

(defun session-fold (session r)
  "FOLD-FLAT-TABLE of every table by the round's challenge R (src/sumcheck.lisp:562)."
  (with-sap (sap r)
    (check (%sumcheck-fold (session-handle session) sap))))

(defun session-run (session state)
  "Every round back to back on the device, from the transcript's B3S STATE after the header
(src/blake3.lisp:127-132): returns the messages (n points D) and the challenges (n D) as flat vectors.  The
pending block handed over must be zero beyond USED (a B3S keeps stale bytes there): a cleared copy goes."
  (let* ((n (session-n session))
         (points (session-points session))
         (d (session-d session))
         (messages (u32-vector (* n points d)))
         (challenges (u32-vector (* n d)))
         (state (b3s-copy state))
         (cv (slot-value state 'exacta.blake3::cv))
         (block (slot-value state 'exacta.blake3::block))
         (used (slot-value state 'exacta.blake3::used))
         (counter (slot-value state 'exacta.blake3::counter)))
    (fill block 0 :start used)
    (sb-sys:with-pinned-objects (cv block messages challenges)
      (check (%sumcheck-run (session-handle session) (sb-sys:vector-sap cv) (sb-sys:vector-sap block) used counter
                            (sb-sys:vector-sap messages) (sb-sys:vector-sap challenges))))
    (values messages challenges)))

(defun finish-session (session names)
  "The read-back at the end of PROVE (src/sumcheck.lisp:564-571): the finals alist (variable . EXT, block 0)
and the folded alist (variable . vector of the K blocks' EXTs).  Ends the session."
  (let* ((d (session-d session))
         (nt (session-tables session))
         (k (session-blocks session))
         (finals (u32-vector (* nt d)))
         (folded (loop repeat nt collect (u32-vector (* k d))))
         (pointers (make-alien system-area-pointer (max nt 1))))
    (unwind-protect
         (sb-sys:with-pinned-objects (finals)
           ;; every folded vector stays pinned across the call
           (labels ((call (rest i)
                      (if rest
                          (sb-sys:with-pinned-objects ((car rest))
                            (setf (deref pointers i) (sb-sys:vector-sap (car rest)))
                            (call (cdr rest) (1+ i)))
                          (check (%sumcheck-finish (session-handle session) (sb-sys:vector-sap finals) pointers)))))
             (call folded 0)))
      (free-alien pointers))
    (values (loop for name in names
                  for t-index from 0
                  collect (cons name (subseq finals (* t-index d) (* (1+ t-index) d))))
            (loop for name in names
                  for flat in folded
                  collect (cons name (coerce (loop for b below k collect (subseq flat (* b d) (* (1+ b) d)))
                                             'vector))))))

;;; ------------------------------------------------------------------ PROVE with its loops on the device

(defun prove/hip (tr n statement tables &key eq constants (label "sc") block-weights
                                          (degree (statement-degree statement constants))
                                          (chained t))
  "PROVE (src/sumcheck.lisp:512-571) with the same arguments and values: the round challenges, the finals
alist and the folded alist.  CHAINED (the default, when the message has at most 7 wire points): the device
runs every round's kernel, SEND and CHALLENGE on a copy of TR's hash state, and TR replays the messages
afterwards, drawing the same challenges -- the proof bytes come from TR exactly as before.  Otherwise one
call per round kernel and one per fold, with TR's own SEND and CHALLENGE between them.  The small-value
branch (:535-545) has no counterpart here: its messages are the same field elements as folding's."
  (let* ((d (transcript-degree tr))
         (points (max degree 1))
         (names (mapcar #'car tables))
         (blocks (if block-weights (length block-weights) 1))
         (handles (mapcar (lambda (entry) (upload-table (cdr entry) d)) tables))       ; MAKE-TABLE, :531
         (stmt (compile-statement statement names (mapcar #'car constants)))
         (rhos '()))
    (unwind-protect
         (let ((session (begin-session stmt d n handles eq block-weights (mapcar #'cdr constants) degree)))
           (absorb tr (header label n degree blocks))                                   ; :534, unchanged
           (if (and chained (<= points 7) (plusp n))
               (multiple-value-bind (messages challenges) (session-run session (transcript-state tr))
                 (dotimes (j n)
                   (let ((row (make-array (list points d) :element-type '(unsigned-byte 32))))
                     (dotimes (i (* points d))
                       (setf (row-major-aref row i) (aref messages (+ (* j points d) i))))
                     (send tr row))                                                     ; :560, the same bytes
                   (let ((r (challenge tr)))                                            ; :561
                     (unless (equalp r (subseq challenges (* j d) (* (1+ j) d)))
                       (error 'device-error :status -7
                                            :message "the device's transcript drew another challenge"))
                     (push r rhos))))
               (dotimes (j n)
                 (send tr (session-round session))                                      ; :556, :560
                 (let ((r (challenge tr)))
                   (session-fold session r)                                             ; :562
                   (push r rhos))))
           (multiple-value-bind (finals folded) (finish-session session names)         ; :564-571
             (values (nreverse rhos) finals folded)))
      (free-statement stmt)
      (mapc #'free-table handles))))

;;; ------------------------------------------------------------------ the other kernels, one call each

(defun rs-encode/hip (messages-handle ncols c)
  "ENCODE (src/rs.lisp:75-85) of NCOLS columns of 2^C base values on the device -> a codewords handle."
  (with-alien ((out (unsigned 64)))
    (check (%rs-encode messages-handle ncols c (addr out)))
    out))

(defun merkle-commit/hip (codewords-handle ncols c)
  "The leaf digests and Merkle levels of a class's codewords (src/pcs.lisp:275-277, 293-302): returns the
levels' handle and the cap as a list of 32-octet vectors."
  (let ((cap (make-array (* 32 128) :element-type '(unsigned-byte 8))))
    (with-alien ((levels (unsigned 64)) (rows (unsigned 64)))
      (with-sap (sap cap)
        (check (%merkle-commit codewords-handle ncols c (addr levels) sap (addr rows))))
      (values levels (loop for i below rows collect (subseq cap (* 32 i) (* 32 (1+ i))))))))

(defun rs-fold/hip (codeword-handle d m n-domain level r)
  "RS:FOLD (src/rs.lisp:93-101) of an extension codeword of 2 M elements on twiddle level LEVEL."
  (with-alien ((out (unsigned 64)))
    (with-sap (sap r)
      (check (%rs-fold codeword-handle d m n-domain level sap (addr out))))
    out))

(defun gkr-reduce-layer/hip (p-handle q-handle d k m)
  "One in-block layer of FRACTION-TREES (src/gkr.lisp:157-170): children (b, x) and (b, x + 2^M)."
  (with-alien ((out-p (unsigned 64)) (out-q (unsigned 64)))
    (check (%gkr-reduce-layer p-handle q-handle d k m (addr out-p) (addr out-q)))
    (values out-p out-q)))

(defun combine-columns/hip (columns-handle ncols len coefficients d)
  "COMBINE-COLUMNS (src/pcs.lisp:434-441) over columns already on the device -> a handle of LEN EXTs."
  (let ((flat (flatten-exts coefficients d)))
    (with-alien ((out (unsigned 64)))
      (with-sap (sap flat)
        (check (%combine-columns columns-handle ncols len d sap (addr out))))
      out)))

(defun dot-pairs/hip (e-handle v-handle)
  "DOT-PAIRS (src/pcs.lisp:473-483) at the parities 0, 1, 2 in one call: three EXT8s."
  (let ((out (u32-vector 24)))
    (with-sap (sap out)
      (check (%dot-pairs e-handle v-handle sap)))
    (loop for parity below 3 collect (subseq out (* 8 parity) (* 8 (1+ parity))))))

(defun fold-table/hip (table-handle r)
  "FOLD-TABLE (src/field.lisp:365-370) of a device table by R -> a handle of half the length."
  (with-alien ((out (unsigned 64)))
    (with-sap (sap r)
      (check (%fold-table table-handle sap (addr out))))
    out))
