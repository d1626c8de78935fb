// A native consumer of the C ABI: the save -> query -> load cycle of
// pegaflow-core's engine tests (tests/engine_basic.rs, hybrid_groups.rs) driven
// from C++ with nothing but include/pegahip.h and the HIP runtime, over both
// transfer modes, both worker forms (block ids / descriptors), blockwise
// allocation, page-first pages small (zero-copy) and large (whole-page
// staging), a 20-layer task whose load is converted in two parts, and 160 MiB
// layers through every worker form.
// Built by `make -C pegaflow_amd/csrc native-tests`; run by
// tests/test_gpu_native.py.  Exit status 0 and a last line "all ok" = pass.
#include "../../include/pegahip.h"
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>
#define OK(x) do{int st_=(x); if(st_!=0){printf("FAIL line %d: %s -> %d %s\n",__LINE__,#x,st_,pf_last_error()); return 1;}}while(0)
int run(bool page_first,int mode,bool desc,bool blockwise,int nseg,int L,uint64_t nb,uint64_t seg,uint64_t n,uint64_t pool_mb){
  printf("case page_first=%d mode=%d desc=%d blockwise=%d nseg=%d L=%d nb=%llu seg=%llu n=%llu\n",page_first,mode,desc,blockwise,nseg,L,(unsigned long long)nb,(unsigned long long)seg,(unsigned long long)n); fflush(stdout);
  pf_engine_config cfg; memset(&cfg,0,sizeof cfg); cfg.pool_size=pool_mb<<20; cfg.pool_shards=1; cfg.blockwise_alloc=blockwise; cfg.use_descriptor_backends=desc;
  pf_engine_t e=nullptr; OK(pf_engine_create(&cfg,&e));
  const uint64_t layer_bytes=nseg*nb*seg;
  std::vector<void*> src(L),dst(L); std::vector<std::vector<uint8_t>> host(L);
  std::mt19937_64 rng(7);
  for(int l=0;l<L;l++){ if(hipMalloc(&src[l],layer_bytes)||hipMalloc(&dst[l],layer_bytes)) return 2; host[l].resize(layer_bytes); { uint64_t* w8=reinterpret_cast<uint64_t*>(host[l].data()); for(uint64_t k=0;k<layer_bytes/8;k++) w8[k]=rng(); for(uint64_t k=layer_bytes&~7ull;k<layer_bytes;k++) host[l][k]=(uint8_t)rng(); } (void)hipMemcpy(src[l],host[l].data(),layer_bytes,hipMemcpyHostToDevice); (void)hipMemset(dst[l],0,layer_bytes);} 
  std::vector<std::string> names(L); std::vector<const char*> cn(L); for(int l=0;l<L;l++){ names[l]="model.layers."+std::to_string(l)+".attn"; cn[l]=names[l].c_str(); }
  std::vector<uint64_t> sz(L,layer_bytes),nbs(L,nb),bpb(L,seg),kvs(L,nseg==2?nb*seg:0),sg(L,nseg);
  for(int which=0;which<2;which++){
    std::vector<uint64_t> ptrs(L); for(int l=0;l<L;l++) ptrs[l]=(uint64_t)(which?dst[l]:src[l]);
    OK(pf_engine_register_context_layer_batch(e,which?"dst":"src","ns",0,0,0,1,1,L,cn.data(),ptrs.data(),sz.data(),nbs.data(),bpb.data(),kvs.data(),sg.data(),nullptr,nullptr,mode,page_first));
  }
  std::vector<uint64_t> ids(nb); for(uint64_t i=0;i<nb;i++) ids[i]=i; std::shuffle(ids.begin(),ids.end(),rng); ids.resize(n);
  std::vector<int64_t> dids(nb); for(uint64_t i=0;i<nb;i++) dids[i]=i; std::shuffle(dids.begin(),dids.end(),rng); dids.resize(n); if(n>3) dids[1]=-1;
  for(int rep=0;rep<3;rep++){
    std::vector<std::vector<uint8_t>> hs(n); std::vector<const uint8_t*> hp(n); std::vector<uint32_t> hl(n);
    for(uint64_t i=0;i<n;i++){ hs[i].resize(8+ (i%3)); hs[i][0]=rep; memcpy(&hs[i][1],&i,4); hp[i]=hs[i].data(); hl[i]=hs[i].size(); }
    std::vector<pf_layer_save> saves(L); for(int l=0;l<L;l++){ saves[l]={cn[l],ids.data(),hp.data(),hl.data(),n}; }
    OK(pf_engine_batch_save(e,"src",0,0,0,saves.data(),L));
    OK(pf_engine_batch_save(e,"src",0,0,0,saves.data(),L));  // dedupe
    uint64_t hits=0,lease=0; OK(pf_engine_query_prefix(e,"dst",hp.data(),hl.data(),n,&hits,&lease)); if(hits!=n){printf("hits %llu\n",(unsigned long long)hits); return 3;}
    const char* const* groups[1]={cn.data()}; uint64_t gs[1]={(uint64_t)L}; const int64_t* dd[1]={dids.data()};
    pf_task_t t=nullptr; OK(pf_engine_batch_load(e,"dst",0,0,1,groups,gs,lease,dd,n,nullptr,&t));
    pf_task_result r; OK(pf_task_wait(t,-1,&r)); OK(pf_task_destroy(t));
    // verify
    for(int l=0;l<L;l++){ std::vector<uint8_t> got(layer_bytes); (void)hipMemcpy(got.data(),dst[l],layer_bytes,hipMemcpyDeviceToHost);
      uint64_t bad=0;
      for(uint64_t i=0;i<n;i++){ if(dids[i]<0) continue; for(int s=0;s<nseg;s++){ const uint8_t* g=&got[s*nb*seg+dids[i]*seg]; const uint8_t* w=&host[l][s*nb*seg+ids[i]*seg];
        if(memcmp(g,w,seg)){ if(bad++<4){ uint64_t at=0; while(g[at]==w[at]) ++at; uint64_t last=seg-1; while(g[last]==w[last]) --last;
            // whose bytes are these?  another position of this layer, or nothing at all
            long long other=-1; int other_seg=-1; for(uint64_t j=0;j<n&&other<0;j++) for(int t=0;t<nseg;t++) if(!memcmp(g+at,&host[l][t*nb*seg+ids[j]*seg+at],last-at+1)){ other=(long long)j; other_seg=t; break; }
            bool zero=true; for(uint64_t k=at;k<=last;k++) if(g[k]){ zero=false; break; }
            { printf("  dword map from byte %llu (one char per 16-byte lane word, bit i set = dword i differs):", (unsigned long long)(at&~15ull));
              for(uint64_t k=at&~15ull;k<=last;k+=16){ int m=0; for(int d=0;d<4;d++) if(memcmp(g+k+4*d,w+k+4*d,4)) m|=1<<d; printf("%x",m);} printf("\n");
              // does the first differing 16-byte word hold another fragment's bytes at the same offset?
              uint64_t k0=at&~15ull; int d0=0; while(!memcmp(g+k0+4*d0,w+k0+4*d0,4)) ++d0;
              for(int l2=0;l2<L;l2++) for(uint64_t j=0;j<nb;j++) for(int t=0;t<nseg;t++) if(!memcmp(g+k0+4*d0,&host[l2][t*nb*seg+j*seg+k0+4*d0],4)) printf("  first wrong dword equals source layer %d block id %llu segment %d at the same offset\n",l2,(unsigned long long)j,t);
              printf("  first wrong dword %02x%02x%02x%02x wanted %02x%02x%02x%02x\n",g[k0+4*d0],g[k0+4*d0+1],g[k0+4*d0+2],g[k0+4*d0+3],w[k0+4*d0],w[k0+4*d0+1],w[k0+4*d0+2],w[k0+4*d0+3]); }
            printf("MISMATCH rep %d layer %d segment %d pos %llu (src id %llu -> dst id %lld): bytes [%llu, %llu] differ; they are %s (pos %lld seg %d)\n",rep,l,s,(unsigned long long)i,(unsigned long long)ids[i],(long long)dids[i],(unsigned long long)at,(unsigned long long)last, zero?"zero":(other>=0?"another position's":"unknown"),other,other_seg); } } } }
      if(bad){ printf("MISMATCH: %llu fragments of layer %d differ in rep %d\n",(unsigned long long)bad,l,rep); return 4; } }
    if(rep==1) pf_engine_evict_all(e);
  }
  OK(pf_engine_unregister_instance(e,"src")); OK(pf_engine_unregister_instance(e,"dst"));
  OK(pf_engine_destroy(e));
  for(int l=0;l<L;l++){ (void)hipFree(src[l]); (void)hipFree(dst[l]); }
  return 0;
}
int main(){
  int rc=0;
  rc|=run(false,0,false,false,2,4,256,4096,100,64);
  rc|=run(false,1,false,false,2,4,256,4096,100,64);
  rc|=run(false,0,true,false,2,4,256,4096,100,64);
  rc|=run(false,1,true,false,1,3,128,1000,50,64);
  rc|=run(false,0,false,true,2,3,128,4096,40,64);
  rc|=run(true,1,false,false,1,5,128,8192,60,64);
  rc|=run(true,0,false,false,1,5,2048,65536,1500,1200);   // page-first, whole-page staging (>64 MiB)
  rc|=run(false,0,false,false,2,20,4096,32768,2500,4000); // staged, two-part conversion on load
  rc|=run(false,0,false,false,2,12,1024,32768,200,600);   // 12.5 MiB layers: staged in groups that share a slot and a launch
  rc|=run(false,1,false,false,2,8,4096,32768,2500,2000);  // kernel mode at the same size: the engine picks the path, as in direct mode
  rc|=run(false,2,false,false,2,8,4096,32768,2500,2000);  // PF_MODE_ZEROCOPY at the same size: zero-copy both ways
  rc|=run(true,2,false,false,1,5,128,8192,60,64);         // PF_MODE_ZEROCOPY over page-first pages
  rc|=run(false,2,true,false,2,4,256,4096,100,64);        // PF_MODE_ZEROCOPY with per-fragment descriptors: the kernel backend
  rc|=run(false,0,true,false,2,8,4096,32768,2500,2000);   // per-fragment descriptors, direct backend, 40 000 per task
  rc|=run(false,1,true,false,2,8,4096,32768,2500,2000);   // per-fragment descriptors, kernel backend
  printf(rc?"FAILED\n":"all ok\n"); return rc;
}
