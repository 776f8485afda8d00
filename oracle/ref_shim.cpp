/* ref_shim.cpp -- TEST INFRASTRUCTURE ONLY (checker, never the product path).
 *
 * Builds the reference's own CPU backend (-DCUDALM_CPU: cpu_rt.h + cpu_kern.h pasted into
 * cudalm.cu) as a shared library by including the reference translation unit from where it
 * lies, and exports plain-C entry points onto its `static` functions. Nothing from the
 * reference is copied: CUDALM_REF_TU is the absolute path of cudalm.cu, given by the Makefile.
 *
 * The build exists only in a container that mounts the reference; the resulting
 * oracle/_ref/libcudalm_ref.so is git-ignored and is used
 *   (1) to write the golden fixtures under tests/golden/,
 *   (2) to cross-check oracle/qlm_oracle.c on larger seeded inputs,
 *   (3) as the "reference" CPU baseline that bench.py times beside the GPU kernels.
 */
#define main cudalm_reference_main_
#include CUDALM_REF_TU
#undef main

extern "C" {

/* Switch off every reduced-precision path exactly as cuda_init does under CUDALM_CPU
 * (cudalm.cu:6621-6623) and create the (fake) cuBLAS handle the GEMM wrappers use. */
void ref_init(int threads){
    g_fp8gemm=g_fp16=g_fp16gemm=g_h16=g_lane=g_fwd_tc=g_dq_tc=g_dkv_tc=g_moef8=g_tiled=g_sub=g_moe_sb=0;
    g_moe_grp=7;
    if(!CB) cublasCreate(&CB);
    if(threads>0) omp_set_num_threads(threads);
}
int ref_threads(void){ return omp_get_max_threads(); }
int ref_sizeof_span(void){ return (int)sizeof(QSpanD); }

/* ---- qlm.cuh:78-111 integer helpers ---- */
unsigned ref_qhashu(unsigned long long x){ return qhashu(x); }
int ref_qsri(float v,unsigned long long i,unsigned long long t){ return qsri(v,i,t); }
int ref_qclmp(int v,int lo,int hi){ return qclmp(v,lo,hi); }
int ref_qd_get(const signed char*d,unsigned long long i,int packed){ return qd_get(d,i,packed); }
void ref_qd_set_host(signed char*d,unsigned long long i,int v,int packed){ qd_set_host(d,i,v,packed); }
unsigned long long ref_qd_bytes(unsigned long long nq,int packed){ return qd_bytes(nq,packed); }
void ref_set_qv4(int v){ d_qv4=v; }

/* ---- qlm.cuh:136-178, 377-441 through the CPU twins cpu_kern.h:771-874 ---- */
void ref_encode(const float*P,signed char*d,signed char*r,float*s,const QSpanD*sp,int nspan,
                int group,int dmax,int packed,int ngrp){
    KL(k_qlm_encode,(unsigned)ngrp,group,group)(P,d,r,s,sp,nspan,group,dmax,packed);
}
void ref_render(float*P,const signed char*d,const float*s,const QSpanD*sp,int nspan,int group,
                int packed,int gi_base,int ng){
    KL(k_qlm_render,(unsigned)ng,group)(P,d,s,sp,nspan,group,packed,gi_base);
}
void ref_step(float*P,const float*G,signed char*d,signed char*r,float*s,signed char*m8,float*m8s,
              unsigned char*v8,float*v8s,const QSpanD*sp,int nspan,int group,int dmax,
              float lr,float b1,float b2,float wd,float gscale,const float*gsp,
              float inv_bc1,float inv_sqrt_bc2,int lrmode,unsigned long long t,int adam,
              long long*stat,int packed,int gi_base,int ng){
    qlm_step_launch(P,G,d,r,s,m8,m8s,v8,v8s,sp,nspan,group,dmax,lr,b1,b2,wd,gscale,gsp,
                    inv_bc1,inv_sqrt_bc2,lrmode,t,adam,stat,packed,gi_base,ng);
}
void ref_step_block(float*P,const float*G,signed char*d,signed char*r,float*s,signed char*m8,float*m8s,
              unsigned char*v8,float*v8s,const QSpanD*sp,int nspan,int group,int dmax,
              float lr,float b1,float b2,float wd,float gscale,
              float inv_bc1,float inv_sqrt_bc2,int lrmode,unsigned long long t,int adam,
              long long*stat,int packed,int gi_base,int ng){
    KL(k_qlm_step,(unsigned)ng,group,group)(P,G,d,r,s,m8,m8s,v8,v8s,sp,nspan,group,dmax,
        lr,b1,b2,wd,gscale,inv_bc1,inv_sqrt_bc2,lrmode,t,adam,stat,packed,gi_base);
}
/* cudalm.cu:4472 through its CPU twin cpu_kern.h:620-648 */
void ref_ng_q4_step(float*P,const float*Gc,signed char*d,signed char*r,float*s,signed char*m8,float*m8s,
                    unsigned char*v8,float*v8s,const int*touched,int ntouched,int group,int dmax,
                    float lr,float b1,float b2,float wd,float sref,float inv_bc1,float inv_sqrt_bc2,
                    unsigned long long t,unsigned long long nt,const float*gs){
    KL(k_ng_q4_step,(unsigned)ntouched,group,group)(P,Gc,d,r,s,m8,m8s,v8,v8s,touched,group,dmax,
        lr,b1,b2,wd,sref,inv_bc1,inv_sqrt_bc2,t,nt,gs);
}
/* cudalm.cu:2794, 2811 through their CPU twins cpu_kern.h:533-546 */
void ref_sqsum(const float*G,unsigned long long n,float*part){ KL(k_sqsum,64,TPB)(G,(size_t)n,part); }
void ref_gnorm(const float*part,int nside,int clip_side,float*gs){ KL(k_gnorm,1,1)(part,nside,clip_side,gs); }
void ref_servo(signed char*d,signed char*r,float*s,const QSpanD*sp,int nspan,int group,int dmax,
               float f_hi,float f_lo,int packed,int ngrp){
    KL(k_qlm_servo,(unsigned)ngrp,group,group)(d,r,s,sp,nspan,group,dmax,f_hi,f_lo,packed);
}

/* ---- expert GEMM wrappers cudalm.cu:3133-3256 over cpu_rt.h:178-352 ---- */
void ref_g_ab(const float*A,const float*B,float*C,int M,int K,int N){ g_ab(A,B,C,M,K,N); }
void ref_g_abt_b(const float*A,const float*B,float*C,int M,int K,int N,float beta){ g_abt_b(A,B,C,M,K,N,beta); }
void ref_g_atb(const float*A,const float*B,float*C,int M,int K,int N){ g_atb(A,B,C,M,K,N); }
void ref_mg_ab(const float*A,const float*B,float*C,int M,int K,int N){ mg_ab(A,B,C,M,K,N); }
void ref_mg_abt_b(const float*A,const float*B,float*C,int M,int K,int N,float beta){ mg_abt_b(A,B,C,M,K,N,beta); }
void ref_mg_atb(const float*A,const float*B,float*C,int M,int K,int N){ mg_atb(A,B,C,M,K,N); }
void ref_mg_flush(void){ mg_flush(); }

/* ---- MoE glue, CPU twins cpu_kern.h:376-482 ---- */
void ref_router_topk(const float*rt,float*rprobs,int*assign,float*gate,int N,int E,int K,
                     const float*bias,int bs){
    KL(k_router_topk,nblk(N,TPB),TPB)(rt,rprobs,assign,gate,N,E,K,bias,bs);
}
void ref_gather(const float*src,const int*perm,float*Xp,int N,int D){
    KL(k_gather,nblk((size_t)N*D,TPB),TPB)(src,perm,Xp,N,D);
}
void ref_scatter_gate(const float*yp,const int*perm,const float*gate,float*out,int N,int D){
    KL(k_scatter_gate,nblk((size_t)N*D,TPB),TPB)(yp,perm,gate,out,N,D);
}
void ref_scatter_add(const float*dXp,const int*perm,float*dst,int N,int D){
    KL(k_scatter_add,nblk((size_t)N*D,TPB),TPB)(dXp,perm,dst,N,D);
}
void ref_moe_dgate(const float*dout,const float*yp,const int*perm,const float*gate,
                   float*d_gate,float*dyp,int N,int D){
    KL(k_moe_dgate,N,TPB)(dout,yp,perm,gate,d_gate,dyp,N,D);
}
void ref_swiglu(const float*G,const float*U,float*O,size_t n){ e_swig(G,U,O,n); }
void ref_swiglu_bwd(const float*Gg,const float*U,const float*dact,float*dg,float*du,size_t n){
    KL(k_swiglu_bwd,nblk(n,TPB),TPB)(Gg,U,dact,dg,du,n);
}
float ref_relerr(const float*a,const float*b,size_t n){ return relerr(a,b,n); }

/* ---- cudalm.cu:638-656, 688-696: the q4n wire format (qtype 3) ---- */
size_t ref_q4n_quantize(const float*P,size_t n,int group,unsigned char*out,size_t cap){
    size_t len=0; uint8_t*q=quantize_params(P,n,3,group,&len);
    if(len<=cap) memcpy(out,q,len);
    free(q); return len;
}
int ref_q4n_dequantize(const unsigned char*buf,size_t len,float*P,size_t n,int group){
    Rd r; r.p=buf; r.end=buf+len; return dequantize_params(&r,P,n,3,group);
}

/* ---- qlm.cuh:702-788: the .opt.q checkpoint, written and read by the reference's own functions over a Qlm
 * put together from host arrays (under CUDALM_CPU device memory is host memory). `spans` is the span table
 * (qi0/gi0/ngrp/sref as the caller filled them); prev_gn goes through the global the reference uses. ---- */
static void ref_qlm_view(Qlm*q,int dmax,int group,int adam,int packed,QSpanD*spans,int nspan,
                         unsigned long long nfloat,bf16*Mc,bf16*Vc,signed char*d,signed char*r,signed char*m8,
                         unsigned char*v8,float*s,float*m8s,float*v8s){
    memset(q,0,sizeof *q);
    q->on=1; q->dmax=dmax; q->group=group; q->adam=adam; q->packed=packed; q->nspan=nspan;
    q->spanH=spans; q->spanD=(QSpanD*)malloc((size_t)nspan*sizeof(QSpanD));
    for(int i=0;i<nspan;i++){ q->nq+=spans[i].n; q->ngrp+=(unsigned long long)spans[i].ngrp; }
    q->nfloat=nfloat; q->Mc=Mc; q->Vc=Vc; q->d=d; q->r=r; q->m8=m8; q->v8=v8; q->s=s; q->m8s=m8s; q->v8s=v8s;
}
int ref_qlm_save(const char*path,int iter,float prev_gn,int dmax,int group,int adam,int packed,QSpanD*spans,int nspan,
                 unsigned long long nfloat,unsigned short*Mc,unsigned short*Vc,signed char*d,signed char*r,signed char*m8,
                 unsigned char*v8,float*s,float*m8s,float*v8s){
    Qlm*q=(Qlm*)malloc(sizeof(Qlm));
    ref_qlm_view(q,dmax,group,adam,packed,spans,nspan,nfloat,(bf16*)Mc,(bf16*)Vc,d,r,m8,v8,s,m8s,v8s);
    g_prev_gn=prev_gn;
    int ok=qlm_save(q,path,iter);
    free(q->spanD); free(q); return ok;
}
int ref_qlm_load(const char*path,int*iter,float*prev_gn,int dmax,int group,int adam,int packed,QSpanD*spans,int nspan,
                 unsigned long long nfloat,unsigned short*Mc,unsigned short*Vc,signed char*d,signed char*r,signed char*m8,
                 unsigned char*v8,float*s,float*m8s,float*v8s){
    Qlm*q=(Qlm*)malloc(sizeof(Qlm));
    ref_qlm_view(q,dmax,group,adam,packed,spans,nspan,nfloat,(bf16*)Mc,(bf16*)Vc,d,r,m8,v8,s,m8s,v8s);
    g_prev_gn=*prev_gn;
    int ok=qlm_load(q,path,iter);
    *prev_gn=g_prev_gn;
    free(q->spanD); free(q); return ok;
}

} /* extern "C" */
