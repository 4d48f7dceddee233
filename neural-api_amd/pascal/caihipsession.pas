{
  caihipsession.pas - the step-resident decode session of libcaihip.so behind the interface the chat engine uses of
  TNNetStreamingDecoder (neural/neuraldecode.pas:1210-1333: StepForward 5696-5712, TruncateTo 5714, Snapshot / Restore
  5759-5843, EnableInt8KVCache 1277-1290, EnableEviction 1257-1276) and of its own generation loop
  (neural/neuralchatengine.pas:1428-1561).

  The session owns a device-resident decoder (weights, KV cache, captured step graphs); the host keeps token ids and, when a
  sampler needs them, one logits row.  Every method maps to ONE entry point of include/caihip.h; errors are raised as
  ECaiHip with the library's own message (cai_last_error), which is what the OpenCL offload object logs through ErrorProc.

  Not compiled in this repository (no fpc in the build image).  tests/test_abi_symbols.py checks that every cai_* call below
  names an external of caihip.pas and passes as many arguments as the external declares.
}
unit caihipsession;

{$mode objfpc}{$H+}

interface

uses
  SysUtils, caihip;

type
  ECaiHip = class(Exception);

  TCaiLongIntArray = array of LongInt;
  TCaiSingleArray = array of Single;

  { One sequence (index 0) of a decoder created from a GGUF file or assembled by the caller. }
  TCaiHipSession = class
  private
    FDec: TCaiDecoder;
    FCfg: TCaiDecoderConfig;
    FSnap: TCaiKVSnap;
    FLogits: TCaiSingleArray;
    FWindowLogits: TCaiSingleArray;
    FLastRow: LongInt;           // the logits row of the last token fed: 0 after a step, Count - 1 after StepWindow
    procedure Check(rc: LongInt; const Where: string);
    function GetPosition: LongInt;
  public
    // EnableHIP analogue of the chat terminal's --gpu branch (neural/neuralchatengine.pas:1156-1157): returns false when
    // no gfx950 device answers, and the caller stays on its CPU path
    class function DeviceAvailable(DeviceOrdinal: LongInt = 0): Boolean;
    // the library reads the file itself (llama / qwen2 architectures; block types stay quantized on the device)
    constructor CreateFromGGUF(const FileName: string; MaxCtx: LongInt; KVInt8: Boolean);
    // a decoder the caller has filled through cai_decoder_set_weight / cai_decoder_set_vector
    constructor CreateFromDecoder(ADecoder: TCaiDecoder);
    destructor Destroy; override;

    // StepForward: one token at the session's position; Logits receives the row of vocab floats when WantLogits.
    // Returns the arg-max token (lowest index on ties: neural/neuralchatengine.pas:683-697).
    function StepForward(Token: LongInt; WantLogits: Boolean): LongInt;
    // prompt ingestion through the matrix-core kernels; returns the arg-max of the last prompt token
    function Prefill(const Tokens: TCaiLongIntArray; First, Count: LongInt; WantLogits: Boolean): LongInt;
    // greedy fast path: MaxNew tokens fed back on the device (neural/neuralchatengine.pas:1493-1494)
    function GenerateGreedy(FirstToken, MaxNew: LongInt): TCaiLongIntArray;
    // width-n window (n <= 8) at the session's position: the verify pass of speculative decoding (StepForward on a width-K
    // twin, neural/neuraldecode.pas:1151-1183).  ArgMax[r] is the model's token after Tokens[First + r]; the logits rows go
    // to WindowLogits when WantLogits.  The caller commits a prefix with TruncateTo.
    procedure StepWindow(const Tokens: TCaiLongIntArray; First, Count: LongInt; WantLogits: Boolean; out ArgMax: TCaiLongIntArray);
    // DecodePromptLookup on the cached session (neural/neuraldecode.pas:7767-7866): Context[0 .. n-2] must be in the cache;
    // returns MaxNew greedy tokens, Passes receives the number of window steps taken
    function GenerateLookup(const Context: TCaiLongIntArray; MatchLen, NumDraft, MaxNew: LongInt; out Passes: LongInt): TCaiLongIntArray;
    // the sampled branch without the logits read-back: the M most probable candidates after the penalties and the
    // temperature, sorted (neural/neuralchatengine.pas:1495-1501), over the row of the last token fed; the random draw stays on the host
    function Candidates(const HistIds, HistCounts: TCaiLongIntArray; Repetition, Frequency, Presence, Temperature: Single;
      M: LongInt; out Tokens: TCaiLongIntArray; out Probs: TCaiSingleArray): LongInt;

    procedure TruncateTo(NewLength: LongInt);          // prefix reuse (neural/neuralchatengine.pas:1434-1439)
    procedure Reset;                                   // after an exception (1630-1636)
    procedure Snapshot;
    procedure Restore;
    procedure EnableInt8KVCache;                       // on a fresh session only, like the reference
    procedure DisableInt8KVCache;                      // back to fp32 rows (neural/neuraldecode.pas:1290), fresh session only
    procedure EnableEviction(SinkTokens, RecentWindow: LongInt);
    procedure DisableEviction;
    function CacheRows(LayerIdx: LongInt): LongInt;    // SDPACacheLength(Index)
    // HiddenState: the input of the vocabulary projection for a row of the last step or window (d_model values)
    function HiddenState(Row: LongInt = 0): TCaiSingleArray;

    property Position: LongInt read GetPosition;
    property VocabSize: LongInt read FCfg.vocab;
    property Logits: TCaiSingleArray read FLogits;
    property WindowLogits: TCaiSingleArray read FWindowLogits;   // [Count][VocabSize] of the last StepWindow
    property Decoder: TCaiDecoder read FDec;
  end;

implementation

procedure TCaiHipSession.Check(rc: LongInt; const Where: string);
var
  Buf: array[0..1023] of AnsiChar;
begin
  if rc = CAI_OK then exit;
  Buf[0] := #0;
  cai_last_error(@Buf[0], 1024);
  raise ECaiHip.CreateFmt('%s: %s (code %d)', [Where, string(PAnsiChar(@Buf[0])), rc]);
end;

class function TCaiHipSession.DeviceAvailable(DeviceOrdinal: LongInt): Boolean;
begin
  Result := cai_init(DeviceOrdinal) = CAI_OK;
end;

constructor TCaiHipSession.CreateFromGGUF(const FileName: string; MaxCtx: LongInt; KVInt8: Boolean);
var
  KV: LongInt;
begin
  inherited Create;
  if KVInt8 then KV := CAI_KV_I8 else KV := CAI_KV_F32;
  Check(cai_decoder_load_gguf(PChar(FileName), MaxCtx, 1, KV, @FDec), 'cai_decoder_load_gguf');
  Check(cai_decoder_get_config(FDec, @FCfg), 'cai_decoder_get_config');
  SetLength(FLogits, FCfg.vocab);
end;

constructor TCaiHipSession.CreateFromDecoder(ADecoder: TCaiDecoder);
begin
  inherited Create;
  FDec := ADecoder;
  Check(cai_decoder_get_config(FDec, @FCfg), 'cai_decoder_get_config');
  SetLength(FLogits, FCfg.vocab);
end;

destructor TCaiHipSession.Destroy;
begin
  if FSnap <> nil then cai_kv_snap_destroy(FSnap);
  if FDec <> nil then cai_decoder_destroy(FDec);
  inherited Destroy;
end;

function TCaiHipSession.GetPosition: LongInt;
begin
  Result := 0;
  Check(cai_decoder_len(FDec, 0, @Result), 'cai_decoder_len');
end;

function TCaiHipSession.StepForward(Token: LongInt; WantLogits: Boolean): LongInt;
var
  Pos: LongInt;
  Row: PSingle;
begin
  Pos := GetPosition;
  if WantLogits then Row := @FLogits[0] else Row := nil;
  Result := -1;
  Check(cai_decoder_step(FDec, @Token, @Pos, 1, Row, @Result), 'cai_decoder_step');
  FLastRow := 0;
end;

function TCaiHipSession.Prefill(const Tokens: TCaiLongIntArray; First, Count: LongInt; WantLogits: Boolean): LongInt;
var
  Row: PSingle;
begin
  Result := -1;
  if Count <= 0 then exit;
  if WantLogits then Row := @FLogits[0] else Row := nil;
  Check(cai_decoder_prefill(FDec, 0, @Tokens[First], Count, GetPosition, Row, @Result), 'cai_decoder_prefill');
  FLastRow := 0;
end;

function TCaiHipSession.GenerateGreedy(FirstToken, MaxNew: LongInt): TCaiLongIntArray;
begin
  SetLength(Result, MaxNew);
  if MaxNew <= 0 then exit;
  Check(cai_decoder_generate(FDec, FirstToken, GetPosition, MaxNew, @Result[0]), 'cai_decoder_generate');
  FLastRow := 0;
end;

procedure TCaiHipSession.StepWindow(const Tokens: TCaiLongIntArray; First, Count: LongInt; WantLogits: Boolean;
  out ArgMax: TCaiLongIntArray);
var
  Rows: PSingle;
begin
  SetLength(ArgMax, Count);
  if Count <= 0 then exit;
  Rows := nil;
  if WantLogits then
  begin
    SetLength(FWindowLogits, Count * FCfg.vocab);
    Rows := @FWindowLogits[0];
  end;
  Check(cai_decoder_step_window(FDec, 0, @Tokens[First], Count, GetPosition, Rows, @ArgMax[0]), 'cai_decoder_step_window');
  FLastRow := Count - 1;
end;

function TCaiHipSession.GenerateLookup(const Context: TCaiLongIntArray; MatchLen, NumDraft, MaxNew: LongInt;
  out Passes: LongInt): TCaiLongIntArray;
begin
  Passes := 0;
  SetLength(Result, MaxNew);
  if (MaxNew <= 0) or (Length(Context) = 0) then exit;
  Check(cai_decoder_generate_lookup(FDec, @Context[0], Length(Context), MatchLen, NumDraft, MaxNew, @Result[0], @Passes),
    'cai_decoder_generate_lookup');
end;

function TCaiHipSession.Candidates(const HistIds, HistCounts: TCaiLongIntArray; Repetition, Frequency, Presence,
  Temperature: Single; M: LongInt; out Tokens: TCaiLongIntArray; out Probs: TCaiSingleArray): LongInt;
var
  PIds, PCounts: PLongInt;
begin
  SetLength(Tokens, M);
  SetLength(Probs, M);
  Result := 0;
  if Length(HistIds) > 0 then begin PIds := @HistIds[0]; PCounts := @HistCounts[0]; end
  else begin PIds := nil; PCounts := nil; end;
  Check(cai_decoder_candidates(FDec, FLastRow, PIds, PCounts, Length(HistIds), Repetition, Frequency, Presence, Temperature, M,
    @Tokens[0], @Probs[0], @Result), 'cai_decoder_candidates');
  SetLength(Tokens, Result);
  SetLength(Probs, Result);
end;

procedure TCaiHipSession.TruncateTo(NewLength: LongInt);
begin
  Check(cai_decoder_truncate(FDec, 0, NewLength), 'cai_decoder_truncate');
end;

procedure TCaiHipSession.Reset;
begin
  Check(cai_decoder_reset(FDec, 0), 'cai_decoder_reset');
end;

procedure TCaiHipSession.Snapshot;
begin
  if FSnap <> nil then begin cai_kv_snap_destroy(FSnap); FSnap := nil; end;
  Check(cai_decoder_snapshot(FDec, 0, @FSnap), 'cai_decoder_snapshot');
end;

procedure TCaiHipSession.Restore;
begin
  if FSnap = nil then raise ECaiHip.Create('Restore without a Snapshot');
  Check(cai_decoder_restore(FDec, 0, FSnap), 'cai_decoder_restore');
end;

procedure TCaiHipSession.EnableInt8KVCache;
begin
  Check(cai_decoder_set_kv_dtype(FDec, CAI_KV_I8), 'cai_decoder_set_kv_dtype');
end;

procedure TCaiHipSession.DisableInt8KVCache;
begin
  Check(cai_decoder_set_kv_dtype(FDec, CAI_KV_F32), 'cai_decoder_set_kv_dtype');
end;

procedure TCaiHipSession.EnableEviction(SinkTokens, RecentWindow: LongInt);
begin
  Check(cai_decoder_set_eviction(FDec, SinkTokens, RecentWindow), 'cai_decoder_set_eviction');
end;

procedure TCaiHipSession.DisableEviction;
begin
  Check(cai_decoder_set_eviction(FDec, 0, 0), 'cai_decoder_set_eviction');
end;

function TCaiHipSession.HiddenState(Row: LongInt): TCaiSingleArray;
begin
  SetLength(Result, FCfg.d_model);
  Check(cai_decoder_hidden_state(FDec, Row, @Result[0]), 'cai_decoder_hidden_state');
end;

function TCaiHipSession.CacheRows(LayerIdx: LongInt): LongInt;
begin
  Result := 0;
  Check(cai_decoder_cache_rows(FDec, 0, LayerIdx, @Result), 'cai_decoder_cache_rows');
end;

end.
